//! src/blas/axpy.zig on libwekua_hip -- the body that replaces src/blas/axpy.zig:102-168 (kernel
//! lookup, setArg, enqueueNdRange).  Signature and shape check as in the reference (axpy.zig:93-100).
//! NOT COMPILED (no Zig toolchain in the build image).
//!
//! `getKernel` and `isSubstracting` (axpy.zig:15-91) are deleted: the library classifies alpha itself
//! (absent -> y += x; -1 -> y -= x, for complex also (-1, -1) as the reference does; else y += alpha*x).
const core = @import("core");
const hip = core.hip;
const Pipeline = core.Pipeline;

const tensor_module = @import("tensor");
const Tensor = tensor_module.Tensor;
const TensorErrors = tensor_module.Errors;

pub fn axpy(
    comptime T: type,
    pipeline: *Pipeline,
    x: *Tensor(T),
    alpha: ?T,
    y: *Tensor(T),
) TensorErrors!void {
    try tensor_module.helpers.eqlTensorsShape(T, x, y);

    const shape3 = [3]u64{ x.depth(), x.rows(), x.cols() };
    const alpha_ptr: ?*const anyopaque = if (alpha) |*a| @ptrCast(a) else null;
    try hip.check(hip.wk_axpy(
        pipeline.command_queue.stream,
        @intCast(core.types.getTypeIndex(T)),
        &shape3,
        x.buffer,
        x.memory_layout.row_pitch,
        x.memory_layout.slice_pitch,
        y.buffer,
        y.memory_layout.row_pitch,
        y.memory_layout.slice_pitch,
        alpha_ptr,
    ));
    try pipeline.append(1);
}
