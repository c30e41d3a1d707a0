//! memory.readFromBuffer / writeToBuffer on libwekua_hip -- the bodies that replace
//! src/tensor/memory/read_from_buffer.zig:13-63 (cl.buffer.writeRect) and write_to_buffer.zig:13-63
//! (cl.buffer.readRect): one pitched copy of the logical region each, asynchronous on the
//! pipeline's stream.  NOT COMPILED (no Zig toolchain in the build image).
const core = @import("core");
const hip = core.hip;
const Pipeline = core.Pipeline;
const tensor_module = @import("main.zig");
const Tensor = tensor_module.Tensor;
const Errors = tensor_module.Errors;

/// HOST -> DEVICE.  `buffer` must stay valid until the pipeline has been waited for.
pub fn readFromBuffer(comptime T: type, pipeline: *Pipeline, tensor: *Tensor(T), buffer: []const T) Errors!void {
    if (buffer.len != tensor.dimensions.number_of_elements_without_padding) return Errors.InvalidBuffer;
    const width = tensor.cols() * @sizeOf(T);
    const rows = tensor.rows();
    try hip.check(hip.wk_copy_h2d_rect_async(
        pipeline.command_queue.stream,
        tensor.buffer,
        tensor.memory_layout.row_pitch * @sizeOf(T),
        tensor.memory_layout.slice_pitch * @sizeOf(T),
        @ptrCast(buffer.ptr),
        width,
        width * rows,
        width,
        rows,
        tensor.depth(),
    ));
    try pipeline.append(1);
}

/// DEVICE -> HOST.
pub fn writeToBuffer(comptime T: type, pipeline: *Pipeline, tensor: *Tensor(T), buffer: []T) Errors!void {
    if (buffer.len != tensor.dimensions.number_of_elements_without_padding) return Errors.InvalidBuffer;
    const width = tensor.cols() * @sizeOf(T);
    const rows = tensor.rows();
    try hip.check(hip.wk_copy_d2h_rect_async(
        pipeline.command_queue.stream,
        @ptrCast(buffer.ptr),
        width,
        width * rows,
        tensor.buffer,
        tensor.memory_layout.row_pitch * @sizeOf(T),
        tensor.memory_layout.slice_pitch * @sizeOf(T),
        width,
        rows,
        tensor.depth(),
    ));
    try pipeline.append(1);
}
