//! src/core/hip.zig -- the binding of libwekua_hip (include/wekua_hip.h) for wekua's Zig modules.
//!
//! Takes the place of the `opencl` import on the gemm / axpy path: every `cl.*` call of src/core,
//! src/tensor and src/blas becomes one of the `extern fn`s below (the files next to this one hold the
//! rewritten bodies).  One declaration per
//! function of the header, same order of parameters.  NOT COMPILED: the image this was written in has
//! no Zig toolchain; a test checks names and parameter counts against the header.
const tensor = @import("../tensor/main.zig");

pub const Props = extern struct {
    name: [64]u8,
    arch: [32]u8,
    ordinal: c_int,
    compute_units: c_int,
    wavefront_size: c_int,
    max_work_group_size: c_int,
    local_mem_bytes: u64,
    global_mem_bytes: u64,
    cache_line_size: c_int,
    clock_mhz: c_int,
};

pub const Device = opaque {};
pub const Stream = opaque {};
pub const Event  = opaque {};

pub extern fn wk_strerror(code: c_int) [*:0]const u8;
pub extern fn wk_abi_version() c_int;
pub extern fn wk_dtype_size(dtype: c_int) usize;
pub extern fn wk_device_count(out_count: *c_int) c_int;
pub extern fn wk_device_open(ordinal: c_int, out: *?*Device) c_int;
pub extern fn wk_device_close(dev: *Device) void;
pub extern fn wk_device_props(dev: *Device, out: *Props) c_int;
pub extern fn wk_stream_create(dev: *Device, out: *?*Stream) c_int;
pub extern fn wk_stream_destroy(s: *Stream) void;
pub extern fn wk_stream_sync(s: *Stream) c_int;
pub extern fn wk_stream_native(s: *Stream) ?*anyopaque;   // the hipStream_t
pub extern fn wk_event_create(dev: *Device, out: *?*Event) c_int;
pub extern fn wk_event_record(e: *Event, s: *Stream) c_int;
pub extern fn wk_event_sync(e: *Event) c_int;
pub extern fn wk_event_destroy(e: *Event) void;
pub extern fn wk_event_elapsed_ms(start: *Event, stop: *Event, out_ms: *f32) c_int;
pub extern fn wk_malloc(dev: *Device, bytes: usize, out: *?*anyopaque) c_int;
pub extern fn wk_free(dev: *Device, ptr: ?*anyopaque) c_int;
pub extern fn wk_mem_info(dev: *Device, free_bytes: *usize, total_bytes: *usize) c_int;
pub extern fn wk_memset_async(s: *Stream, ptr: *anyopaque, byte: c_int, bytes: usize) c_int;
pub extern fn wk_copy_h2d_rect_async(s: *Stream, dst: *anyopaque, dst_row_pitch: usize, dst_slice_pitch: usize,
    host_src: *const anyopaque, src_row_pitch: usize, src_slice_pitch: usize,
    width_bytes: usize, rows: usize, slices: usize) c_int;
pub extern fn wk_copy_d2h_rect_async(s: *Stream, host_dst: *anyopaque, dst_row_pitch: usize, dst_slice_pitch: usize,
    src: *const anyopaque, src_row_pitch: usize, src_slice_pitch: usize,
    width_bytes: usize, rows: usize, slices: usize) c_int;
pub extern fn wk_copy_d2d_rect_async(s: *Stream, dst: *anyopaque, dst_row_pitch: usize, dst_slice_pitch: usize,
    src: *const anyopaque, src_row_pitch: usize, src_slice_pitch: usize,
    width_bytes: usize, rows: usize, slices: usize) c_int;
pub extern fn wk_fill(s: *Stream, dtype: c_int, ptr: *anyopaque, shape3: *const [3]u64,
    row_pitch: u64, slice_pitch: u64, host_scalar: *const anyopaque) c_int;
pub extern fn wk_identity(s: *Stream, dtype: c_int, ptr: *anyopaque, size: u64, pitch_sum: u64) c_int;
pub extern fn wk_axpy(s: *Stream, dtype: c_int, shape3: *const [3]u64,
    x: *const anyopaque, x_row_pitch: u64, x_slice_pitch: u64,
    y: *anyopaque, y_row_pitch: u64, y_slice_pitch: u64, host_alpha: ?*const anyopaque) c_int;
pub extern fn wk_gemm(s: *Stream, dtype: c_int, op_a: c_int, op_b: c_int, m: u64, n: u64, k: u64,
    host_alpha: ?*const anyopaque, a: *const anyopaque, lda: u64, b: *const anyopaque, ldb: u64,
    host_beta: ?*const anyopaque, c: *anyopaque, ldc: u64, workspace: ?*anyopaque, workspace_bytes: usize) c_int;
/// the same call for a B that is still packed in the workspace from the previous call (optional; see the PackedTensors row)
pub extern fn wk_gemm_packed_b_kept(s: *Stream, dtype: c_int, op_a: c_int, op_b: c_int, m: u64, n: u64, k: u64,
    host_alpha: ?*const anyopaque, a: *const anyopaque, lda: u64, b: *const anyopaque, ldb: u64,
    host_beta: ?*const anyopaque, c: *anyopaque, ldc: u64, workspace: ?*anyopaque, workspace_bytes: usize) c_int;
pub extern fn wk_gemm_workspace_bytes(dtype: c_int, op_a: c_int, op_b: c_int, m: u64, n: u64, k: u64) usize;

pub const HipError = error{ HipFailure, OutOfMemory, DevicesArrayEmpty, ScratchTooSmall };

/// WK_E_* -> the Zig error the reference already returns at that place.
pub fn check(code: c_int) (tensor.Errors || HipError)!void {
    return switch (code) {
        0 => {},
        1 => error.InvalidValue,          2 => error.InvalidCoordinates,
        3 => error.InvalidBuffer,         4 => error.UnqualTensorsAttribute,
        5 => error.UnqualTensorsShape,    6 => error.UnqualTensorsDimension,
        7 => error.UnqualTensorsContext,  8 => error.OutOfMemory,
        9 => error.TypeNotSupported,      10 => error.DevicesArrayEmpty,
        11 => error.ScratchTooSmall,      else => error.HipFailure,
    };
}

// ---- what one MLP training step needs besides gemm / axpy (src/math, src/nn) ----
pub extern fn wk_hadamard(s: *Stream, dtype: c_int, shape3: *const [3]u64, x: *anyopaque, x_row_pitch: u64, x_slice_pitch: u64,
    y: *const anyopaque, y_row_pitch: u64, y_slice_pitch: u64) c_int;
pub extern fn wk_activation(s: *Stream, dtype: c_int, kind: c_int, shape3: *const [3]u64, x: *anyopaque, row_pitch: u64, slice_pitch: u64) c_int;
pub extern fn wk_activation_dev(s: *Stream, dtype: c_int, kind: c_int, shape3: *const [3]u64, out: *const anyopaque, out_row_pitch: u64,
    out_slice_pitch: u64, dev: *anyopaque, dev_row_pitch: u64, dev_slice_pitch: u64) c_int;
pub extern fn wk_bias_activation(s: *Stream, dtype: c_int, kind: c_int, rows: u64, cols: u64, out: *anyopaque, out_pitch: u64, bias: ?*const anyopaque) c_int;
pub extern fn wk_gemm_bias_activation(s: *Stream, dtype: c_int, op_a: c_int, op_b: c_int, m: u64, n: u64, k: u64, a: *const anyopaque, lda: u64, b: *const anyopaque, ldb: u64, c: *anyopaque, ldc: u64, bias: ?*const anyopaque, kind: c_int) c_int;
pub extern fn wk_bias_step(s: *Stream, dtype: c_int, rows: u64, cols: u64, sens: *const anyopaque, pitch: u64, bias_grad: *anyopaque) c_int;
pub extern fn wk_bias_step_static(s: *Stream, dtype: c_int, rows: u64, cols: u64, sens: *const anyopaque, pitch: u64, bias_grad: *anyopaque) c_int;
pub extern fn wk_sensitivity_step(s: *Stream, dtype: c_int, kind: c_int, rows: u64, cols: u64, out: ?*const anyopaque, out_pitch: u64,
    sens: *anyopaque, sens_pitch: u64, dev: *anyopaque, dev_pitch: u64, bias_grad: ?*anyopaque) c_int;
pub extern fn wk_mse(s: *Stream, dtype: c_int, shape3: *const [3]u64, output: *const anyopaque, out_row_pitch: u64, out_slice_pitch: u64,
    expected: *const anyopaque, exp_row_pitch: u64, exp_slice_pitch: u64, err: *anyopaque, err_row_pitch: u64, err_slice_pitch: u64,
    dev: ?*anyopaque, dev_row_pitch: u64, dev_slice_pitch: u64) c_int;
pub extern fn wk_sum_workspace_bytes(dtype: c_int) usize;
pub extern fn wk_sum(s: *Stream, dtype: c_int, shape3: *const [3]u64, x: *const anyopaque, row_pitch: u64, slice_pitch: u64,
    workspace: *anyopaque, dev_result: *anyopaque, scale: f64) c_int;
pub extern fn wk_adam_step(s: *Stream, dtype: c_int, shape3: *const [3]u64, w: *anyopaque, w_row_pitch: u64, w_slice_pitch: u64,
    g: *const anyopaque, g_row_pitch: u64, g_slice_pitch: u64, m: *anyopaque, v: *anyopaque, mv_row_pitch: u64, mv_slice_pitch: u64,
    lr: f64, beta1: f64, beta2: f64, eps: f64, step: u64) c_int;
pub const AdamTensor = extern struct { w: *anyopaque, g: *const anyopaque, m: *anyopaque, v: *anyopaque, shape3: [3]u64,
    w_row_pitch: u64, w_slice_pitch: u64, g_row_pitch: u64, g_slice_pitch: u64, mv_row_pitch: u64, mv_slice_pitch: u64 };
pub extern fn wk_adam_step_multi(s: *Stream, dtype: c_int, count: u32, host_tensors: [*]const AdamTensor,
    lr: f64, beta1: f64, beta2: f64, eps: f64, step: u64) c_int;

// ---- tensor support operations (src/tensor) ----
pub extern fn wk_transpose(s: *Stream, dtype: c_int, ndim: c_int, shape: [*]const u64, src_pitches: [*]const u64,
    dst_pitches: [*]const u64, dim0: c_int, dim1: c_int, src: *const anyopaque, dst: *anyopaque) c_int;
pub extern fn wk_random_uniform(s: *Stream, dtype: c_int, shape3: *const [3]u64, ptr: *anyopaque, row_pitch: u64, slice_pitch: u64,
    seed: u64, host_min: ?*const anyopaque, host_range: ?*const anyopaque) c_int;
pub extern fn wk_to_complex(s: *Stream, real_dtype: c_int, shape3: *const [3]u64, src: *const anyopaque, src_row_pitch: u64,
    src_slice_pitch: u64, dst: *anyopaque, dst_row_pitch: u64, dst_slice_pitch: u64, space: c_int) c_int;
pub extern fn wk_to_real(s: *Stream, real_dtype: c_int, shape3: *const [3]u64, src: *const anyopaque, src_row_pitch: u64,
    src_slice_pitch: u64, dst: *anyopaque, dst_row_pitch: u64, dst_slice_pitch: u64, space: c_int) c_int;
pub extern fn wk_random_hash(index: u64, seed: u64) u64;   // host copy of the device hash, for tests
