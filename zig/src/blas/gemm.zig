//! src/blas/gemm.zig on libwekua_hip -- what replaces src/blas/gemm.zig:60-359 (PackedTensors) and
//! :846-873 (the two branches of `gemm`).  `Operation` (:25-29) and `validateTensors` (:442-485) stay
//! as they are; `getAlgorithm`, the kernel caches, `gemmWithoutPacking` / `gemmWithPacking` and the
//! seven .cl files are no longer used.  NOT COMPILED (no Zig toolchain in the build image).
const std = @import("std");
const core = @import("core");
const hip = core.hip;
const Pipeline = core.Pipeline;
const CommandQueue = core.CommandQueue;

const tensor_module = @import("tensor");
const Tensor = tensor_module.Tensor;
const TensorErrors = tensor_module.Errors;

pub const Operation = enum(u8) { no_transpose = 0, transpose = 1 };

/// Same name, constructors and shape validation as the reference's PackedTensors; instead of two
/// packed tensors it owns one device block that wk_gemm uses as the workspace of its own pack pass
/// (digit planes of the 8/16/32/64-bit integers, the re-formed operands of the complex types; zero
/// bytes for f32 / f64, whose tiles go from the row-major operands straight into LDS).
pub fn PackedTensors(comptime T: type) type {
    return struct {
        const Self = @This();

        allocator: std.mem.Allocator,
        device: *hip.Device,
        n_size: u64, // rows of C
        m_size: u64, // columns of C
        k_size: u64,
        workspace: ?*anyopaque,
        workspace_bytes: usize,
        // optional, beyond the reference: B stays packed while the same tensor comes back
        keep_b: bool = false,
        kept_b_serial: u64 = 0,
        kept_op_b: Operation = .no_transpose,
        kept_alpha: ?T = null,

        pub fn init(pipeline: *Pipeline, result_tensor: *Tensor(T), k_size: u64, vectors_enabled: bool) TensorErrors!*Self {
            const shape = result_tensor.dimensions.shape;
            if (shape.len != 2) return TensorErrors.InvalidValue;
            return initWithDimensions(pipeline, shape[0], shape[1], k_size, .@"2x2", vectors_enabled);
        }

        pub fn initWithDimensions(
            pipeline: *Pipeline,
            n_size: u64,
            m_size: u64,
            k_size: u64,
            recommended_algorithm: tensor_module.GemmAlgorithm,
            vectors_enabled: bool,
        ) TensorErrors!*Self {
            _ = recommended_algorithm; // the library picks its tile per call
            _ = vectors_enabled;
            if (n_size == 0 or m_size == 0 or k_size == 0) return TensorErrors.InvalidValue;
            const context = pipeline.command_queue.context;
            const self = try context.allocator.create(Self);
            errdefer context.allocator.destroy(self);
            const dtype: c_int = @intCast(core.types.getTypeIndex(T));
            const bytes = hip.wk_gemm_workspace_bytes(dtype, 0, 0, n_size, m_size, k_size);
            var block: ?*anyopaque = null;
            if (bytes > 0) try hip.check(hip.wk_malloc(context.device, bytes, &block));
            self.* = .{
                .allocator = context.allocator,
                .device = context.device,
                .n_size = n_size,
                .m_size = m_size,
                .k_size = k_size,
                .workspace = block,
                .workspace_bytes = bytes,
            };
            return self;
        }

        pub fn deinit(self: *Self, pipeline: *Pipeline) void {
            pipeline.waitAndCleanup();
            _ = hip.wk_free(self.device, self.workspace);
            self.allocator.destroy(self);
        }

        /// Shape agreement of a call with this handle (the checks of gemm.zig:195-270).
        pub fn validateTensors(self: *const Self, a: *Tensor(T), op_a: Operation, b: *Tensor(T), op_b: Operation) TensorErrors!void {
            const a_shape = a.dimensions.shape;
            const b_shape = b.dimensions.shape;
            const rows = if (op_a == .transpose) a_shape[1] else a_shape[0];
            const k_a = if (op_a == .transpose) a_shape[0] else a_shape[1];
            const cols = if (op_b == .transpose) b_shape[0] else b_shape[1];
            if (rows != self.n_size or cols != self.m_size or k_a != self.k_size) return TensorErrors.InvalidValue;
        }

        /// The pack pass runs inside wk_gemm; kept so that callers compile unchanged (gemm.zig:272-357).
        pub fn pack(self: *Self, pipeline: *Pipeline, a: *Tensor(T), op_a: Operation, b: *Tensor(T), op_b: Operation) TensorErrors!void {
            _ = pipeline;
            try self.validateTensors(a, op_a, b, op_b);
        }

        pub fn keepB(self: *Self, on: bool) void {
            self.keep_b = on;
            self.kept_b_serial = 0;
        }

        pub fn invalidateB(self: *Self) void {
            self.kept_b_serial = 0;
        }

        fn holdsB(self: *Self, b: *Tensor(T), op_b: Operation, alpha: ?T) bool {
            const same = self.keep_b and self.kept_b_serial == b.serial and self.kept_op_b == op_b and
                std.meta.eql(self.kept_alpha, alpha);
            self.kept_b_serial = if (self.keep_b) b.serial else 0;
            self.kept_op_b = op_b;
            self.kept_alpha = alpha;
            return same;
        }
    };
}

pub fn gemm(
    comptime T: type,
    pipeline: *Pipeline,
    alpha: ?T,
    a: *Tensor(T),
    op_a: Operation,
    b: *Tensor(T),
    op_b: Operation,
    beta: ?T,
    c: *Tensor(T),
    packed_tensors: ?*PackedTensors(T),
) TensorErrors!void {
    try validateTensors(T, a, b, c, op_a, op_b); // gemm.zig:442-485, unchanged

    const a_shape = a.dimensions.shape;
    const c_shape = c.dimensions.shape;
    const k_size = if (op_a == .transpose) a_shape[0] else a_shape[1];
    const alpha_ptr: ?*const anyopaque = if (alpha) |*v| @ptrCast(v) else null;
    const beta_ptr: ?*const anyopaque = if (beta) |*v| @ptrCast(v) else null;

    var workspace: ?*anyopaque = null;
    var workspace_bytes: usize = 0;
    var b_kept = false;
    if (packed_tensors) |p| {
        try p.validateTensors(a, op_a, b, op_b);
        workspace = p.workspace;
        workspace_bytes = p.workspace_bytes;
        b_kept = p.holdsB(b, op_b, alpha);
    }

    const call = if (b_kept) &hip.wk_gemm_packed_b_kept else &hip.wk_gemm;
    try hip.check(call(
        pipeline.command_queue.stream,
        @intCast(core.types.getTypeIndex(T)),
        @intFromEnum(op_a),
        @intFromEnum(op_b),
        c_shape[0],
        c_shape[1],
        k_size,
        alpha_ptr,
        a.buffer,
        a.memory_layout.row_pitch,
        b.buffer,
        b.memory_layout.row_pitch,
        beta_ptr,
        c.buffer,
        c.memory_layout.row_pitch,
        workspace,
        workspace_bytes,
    ));
    try pipeline.append(1);
}

const validateTensors = @import("gemm_validate.zig").validateTensors; // the reference's gemm.zig:442-485 moved out unchanged
