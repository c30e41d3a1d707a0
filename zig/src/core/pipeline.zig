//! src/core/pipeline.zig on a HIP stream -- replaces the event list of the reference's Pipeline
//! (src/core/pipeline.zig:1-80).  NOT COMPILED (no Zig toolchain in the build image).
//!
//! The reference keeps every cl_event an enqueue returned and hands the last batch to the next
//! enqueue as its wait list.  A wk_stream is in order, so no wait lists exist any more: the
//! pipeline only counts what was enqueued since the last wait (callers and tests read
//! `prevEvents()` / `pending()`), and `waitAndCleanup` is one stream synchronisation.
const std = @import("std");
const hip = @import("hip.zig");
const CommandQueue = @import("command_queue.zig");

command_queue: *CommandQueue,
allocator: std.mem.Allocator,
/// enqueues since the last waitAndCleanup (the reference: events.items.len)
pending: usize,
/// size of the last batch appended (the reference: events.items.len - prev_batch_start)
prev_batch: usize,

pub fn init(command_queue: *CommandQueue) error{OutOfMemory}!*Pipeline {
    const allocator = command_queue.context.allocator;
    const self = try allocator.create(Pipeline);
    self.* = .{ .allocator = allocator, .command_queue = command_queue, .pending = 0, .prev_batch = 0 };
    return self;
}

pub fn deinit(self: *Pipeline) void {
    self.allocator.destroy(self);
}

/// Nothing to reserve: kept so that callers compile unchanged.
pub fn prealloc(self: *Pipeline, capacity: usize) error{OutOfMemory}!void {
    _ = self;
    _ = capacity;
}

/// Number of enqueues in the last batch, or null when nothing is pending (the reference returns the
/// slice of events; on an in-order stream only its length still means something).
pub fn prevEvents(self: *Pipeline) ?usize {
    if (self.pending == 0) return null;
    return self.prev_batch;
}

pub fn append(self: *Pipeline, count: usize) error{OutOfMemory}!void {
    self.prev_batch = count;
    self.pending += count;
}

/// src/core/pipeline.zig:47-61: cl.event.waitForMany + release becomes one wk_stream_sync.
pub fn waitAndCleanup(self: *Pipeline) void {
    if (self.pending == 0) return;
    const code = hip.wk_stream_sync(self.command_queue.stream);
    if (code != 0) {
        std.debug.panic("Unexpected error ({s}) while waiting for the stream", .{std.mem.span(hip.wk_strerror(code))});
    }
    self.pending = 0;
    self.prev_batch = 0;
}

pub fn clear(self: *Pipeline) void {
    self.pending = 0;
    self.prev_batch = 0;
}

const Pipeline = @This();
