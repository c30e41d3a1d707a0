//! src/tensor/main.zig on libwekua_hip -- the bodies that replace `Tensor(T).empty / alloc / release`
//! (src/tensor/main.zig:112-277): a hipMalloc'd block with a layout chosen for gfx950 instead of a
//! cl_mem with padded rows and a device copy of the pitches.  The struct's fields (`dimensions`,
//! `memory_layout`, `flags`, `work_configuration`) keep their names and meaning.
//! NOT COMPILED (no Zig toolchain in the build image).
//!
//! Layout: row-major {depth, rows, cols}; row pitch = cols rounded up to the queue's vector width
//! (16 bytes / element size), plus 512 bytes when the pitch is a multiple of 1 KiB and at least 16 KiB
//! (rows 32 KiB apart alias in the memory channels); no padding of the row count; no pitches buffer.
const std = @import("std");
const core = @import("core");
const hip = core.hip;
const Context = core.Context;
const Pipeline = core.Pipeline;

var next_serial = std.atomic.Value(u64).init(1);

pub fn emptyBody(comptime T: type, comptime Self: type, context: *const Context, pipeline: *Pipeline, shape: []const u64, config: anytype) !*Self {
    _ = pipeline;
    if (shape.len == 0) return error.InvalidValue;
    const allocator = context.allocator;
    const tensor = try allocator.create(Self);
    errdefer allocator.destroy(tensor);
    tensor.context = context;
    tensor.serial = next_serial.fetchAdd(1, .monotonic);
    tensor.arena = std.heap.ArenaAllocator.init(allocator);
    errdefer tensor.arena.deinit();
    const arena = tensor.arena.allocator();

    tensor.dimensions.shape = try arena.dupe(u64, shape);
    for (shape) |s| if (s == 0) return error.InvalidValue;

    const is_complex = comptime core.types.isComplex(T);
    const type_id = comptime core.types.getTypeIndex(T);
    var vector_width: u64 = 1;
    if (!is_complex and config.vectors_enabled) vector_width = @intCast(context.command_queues[0].vector_widths[type_id]);
    tensor.flags.vectors_enabled = vector_width > 1;

    const ndim = shape.len;
    const cols = shape[ndim - 1];
    const rows: u64 = if (ndim >= 2) shape[ndim - 2] else 1;
    var depth: u64 = 1;
    for (shape[0 .. ndim -| 2]) |e| depth *= e;

    var row_pitch = cols;
    if (row_pitch % vector_width != 0) row_pitch += vector_width - row_pitch % vector_width;
    const pitch_bytes = row_pitch * @sizeOf(T);
    if (rows * depth > 1 and pitch_bytes >= 16384 and pitch_bytes % 1024 == 0) row_pitch += 512 / @sizeOf(T);

    const vl_shape = try arena.dupe(u64, shape);
    vl_shape[ndim - 1] = row_pitch / vector_width;
    tensor.dimensions.vl_shape = vl_shape;
    tensor.dimensions.number_of_elements_without_padding = depth * rows * cols;
    tensor.memory_layout.row_pitch = row_pitch;
    tensor.memory_layout.row_pitch_for_vectors = row_pitch / vector_width;
    tensor.memory_layout.slice_pitch = row_pitch * rows;
    tensor.memory_layout.slice_pitch_for_vectors = tensor.memory_layout.slice_pitch / vector_width;
    tensor.dimensions.number_of_elements = tensor.memory_layout.slice_pitch * depth;
    tensor.memory_layout.number_of_vectors = tensor.dimensions.number_of_elements / vector_width;
    tensor.memory_layout.size = tensor.dimensions.number_of_elements * @sizeOf(T);

    // element strides of the padded layout, outermost first (main.zig:198-220)
    const pitches = try arena.alloc(u64, ndim);
    pitches[ndim - 1] = 1;
    if (ndim >= 2) pitches[ndim - 2] = row_pitch;
    var p = tensor.memory_layout.slice_pitch;
    var i = ndim -| 2;
    while (i > 0) {
        i -= 1;
        pitches[i] = p;
        p *= shape[i];
    }
    tensor.dimensions.pitches = pitches;

    var block: ?*anyopaque = null;
    try hip.check(hip.wk_malloc(context.device, tensor.memory_layout.size, &block));
    tensor.buffer = block.?;
    return tensor;
}

/// Tensor.alloc = empty + fill.zeroes (main.zig:265-277); fill.zeroes of a whole buffer is one memset.
pub fn allocBody(comptime T: type, comptime Self: type, context: *const Context, pipeline: *Pipeline, shape: []const u64, config: anytype) !*Self {
    const tensor = try emptyBody(T, Self, context, pipeline, shape, config);
    errdefer releaseBody(Self, tensor, pipeline);
    try hip.check(hip.wk_memset_async(pipeline.command_queue.stream, tensor.buffer, 0, tensor.memory_layout.size));
    try pipeline.append(1);
    return tensor;
}

/// Tensor.release drains the pipeline first (main.zig:253-263).
pub fn releaseBody(comptime Self: type, self: *Self, pipeline: *Pipeline) void {
    pipeline.waitAndCleanup();
    _ = hip.wk_free(self.context.device, self.buffer);
    const allocator = self.context.allocator;
    self.arena.deinit();
    allocator.destroy(self);
}
