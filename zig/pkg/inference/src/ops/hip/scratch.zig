//! Grow-only device scratch (ops/cuda/scratch.zig for `hip`): the workspace the small-batch and
//! prefill launchers ask for (quantized activations, partial sums of K shares).  Growing waits
//! for the stream first, because kernels already queued may still be using the old allocation.
const buffer_mod = @import("buffer.zig");
const context_mod = @import("context.zig");
const driver_mod = @import("driver.zig");

pub const DeviceScratch = struct {
    buffer: buffer_mod.DeviceBuffer = .{},

    pub fn deinit(self: *DeviceScratch, ctx: *context_mod.HipContext) void {
        self.buffer.free(ctx);
    }

    pub fn acquire(self: *DeviceScratch, ctx: *context_mod.HipContext, len: usize) driver_mod.Error!buffer_mod.DeviceBuffer {
        if (len == 0) return .{};
        if (self.buffer.len < len) {
            if (self.buffer.ptr != 0) {
                try ctx.synchronize();
                self.buffer.free(ctx);
            }
            // rounded up so that a run of slightly growing requests allocates once
            const rounded = (len + (1 << 20) - 1) & ~@as(usize, (1 << 20) - 1);
            self.buffer = try buffer_mod.DeviceBuffer.alloc(ctx, rounded);
        }
        return .{ .ptr = self.buffer.ptr, .len = len };
    }
};
