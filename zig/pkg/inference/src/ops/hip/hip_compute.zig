//! The `hip` compute backend: ops/cuda/cuda_compute.zig's contract on an MI355X, for the
//! block-quantized matmul path.  Device buffers, the stream and the kernel module are owned
//! here; the kernels run from this backend's code object (one row) or through the C ABI of
//! libantfly_hip_qmatmul on this backend's stream (more rows) -- see kernels.zig.
//!
//! Implemented: tensor plumbing (fromFloat32*, toFloat32, tensorDType/Shape, evalTensor,
//! freeTensor, getWeight), weight ingest from raw GGUF bytes with the device-side repack, and
//! `linearNoBias` / `linearNoBiasPlanned` on Q4_0 / Q8_0 weights.  Every other required entry of
//! the op table answers error.HipOpUnsupported (the CUDA backend does the same for the ops it
//! lacks, cuda_compute.zig:1122-1127).
const std = @import("std");
const ops = @import("../ops.zig");
const tensor_mod = @import("../../tensor.zig");
const gguf_tensor_types = @import("../../gguf/tensor_types.zig");
const weight_source_mod = @import("../../models/weight_source.zig");
const operator_plan_mod = @import("../../graph/operator_plan.zig");
const buffer_mod = @import("buffer.zig");
const context_mod = @import("context.zig");
const kernels_mod = @import("kernels.zig");
const scratch_mod = @import("scratch.zig");

const CT = ops.CT;
const DeviceBuffer = buffer_mod.DeviceBuffer;

/// Same fields as CudaTensor (cuda_compute.zig:29-38) plus how a quantized weight is laid out.
pub const HipTensor = struct {
    buffer: DeviceBuffer,
    dtype: tensor_mod.DType,
    shape: []i64,
    elem_count: usize,
    quant_type: ?gguf_tensor_types.TensorType = null,
    prepared: bool = false, // quantized weight repacked for the kernels (else raw GGUF bytes)
    owns_buffer: bool = true,
    owns_shape: bool = true,
    owned_by_tensor: bool = true,
};

const max_pooled_buffers = 256; // cuda_compute.zig:193-223

pub const HipCompute = struct {
    allocator: std.mem.Allocator,
    ctx: context_mod.HipContext,
    kernels: kernels_mod.KernelModule,
    resident_weights: std.StringHashMapUnmanaged(HipTensor) = .{},
    temp_buffers: std.ArrayListUnmanaged(DeviceBuffer) = .empty,
    workspace: scratch_mod.DeviceScratch = .{},
    owned_by_backend: bool = false,

    pub fn init(allocator: std.mem.Allocator) !HipCompute {
        var ctx = try context_mod.HipContext.initDefault();
        errdefer ctx.deinit();
        const kernels = try kernels_mod.KernelModule.load(&ctx);
        return .{ .allocator = allocator, .ctx = ctx, .kernels = kernels };
    }

    pub fn create(allocator: std.mem.Allocator) !*HipCompute {
        const self = try allocator.create(HipCompute);
        errdefer allocator.destroy(self);
        self.* = try init(allocator);
        self.owned_by_backend = true;
        return self;
    }

    pub fn deinit(self: *HipCompute) void {
        self.ctx.synchronize() catch {};
        var it = self.resident_weights.iterator();
        while (it.next()) |entry| {
            self.allocator.free(entry.key_ptr.*);
            entry.value_ptr.buffer.free(&self.ctx);
            self.allocator.free(entry.value_ptr.shape);
        }
        self.resident_weights.deinit(self.allocator);
        for (self.temp_buffers.items) |*b| b.free(&self.ctx);
        self.temp_buffers.deinit(self.allocator);
        self.workspace.deinit(&self.ctx);
        self.kernels.unload(&self.ctx);
        self.ctx.deinit();
    }

    pub fn computeBackend(self: *HipCompute) ops.ComputeBackend {
        return .{ .ptr = self, .vtable = &vtable };
    }

    /// Raw GGUF bytes go to the device unchanged; Q4_0 / Q8_0 matrices are then repacked on the
    /// device (invisible to callers: `getWeight` hands out the same kind of handle).  Other
    /// quantized types stay resident as raw bytes and are refused at the op, like the CUDA
    /// backend (cuda_compute.zig:116-134, :703-712).
    pub fn insertWeightFromLoaded(self: *HipCompute, owned_key: []const u8, loaded: *const weight_source_mod.LoadedWeight) !void {
        const quant = loaded.quantized_storage orelse return error.UnsupportedTensorType; // dense tensors stay with the host ops
        const raw = quant.raw_bytes;
        const shape = try self.allocator.dupe(i64, quant.shape);
        errdefer self.allocator.free(shape);
        var device = try DeviceBuffer.alloc(&self.ctx, raw.len);
        errdefer device.free(&self.ctx);
        try device.copyFromHost(&self.ctx, raw);
        try self.ctx.synchronize();

        var tensor = HipTensor{
            .buffer = device,
            .dtype = .u8,
            .shape = shape,
            .elem_count = try elementCountFromShape(shape),
            .quant_type = quant.tensor_type,
            .owns_buffer = false,
            .owned_by_tensor = false,
        };
        if (kernelType(quant.tensor_type)) |tt| {
            if (shape.len == 2 and shape[1] > 0 and @mod(shape[1], 32) == 0) {
                const out_dim: usize = @intCast(shape[0]);
                const in_dim: usize = @intCast(shape[1]);
                var prepared = try DeviceBuffer.alloc(&self.ctx, kernels_mod.preparedWeightBytes(tt, out_dim, in_dim));
                errdefer prepared.free(&self.ctx);
                try self.kernels.launchPrepareWeight(&self.ctx, tt, prepared, device, out_dim, in_dim);
                try self.ctx.synchronize();
                device.free(&self.ctx); // the staging copy of the raw bytes is not kept
                tensor.buffer = prepared;
                tensor.prepared = true;
            }
        }
        if (try self.resident_weights.fetchPut(self.allocator, owned_key, tensor)) |old| {
            var old_tensor = old.value;
            old_tensor.buffer.free(&self.ctx);
            self.allocator.free(old_tensor.shape);
            self.allocator.free(old.key);
        }
    }
};

fn kernelType(tensor_type: gguf_tensor_types.TensorType) ?kernels_mod.TensorType {
    return switch (tensor_type) {
        .known => |known| switch (known) {
            .Q4_0 => .q4_0,
            .Q8_0 => .q8_0,
            else => null,
        },
        else => null,
    };
}

fn selfFrom(ctx: *anyopaque) *HipCompute {
    return @ptrCast(@alignCast(ctx));
}

fn tensorFromCt(tensor: CT) *HipTensor {
    return @ptrCast(@alignCast(tensor));
}

fn backendKind(_: *anyopaque) ops.BackendKind {
    return .hip;
}

fn deinitBackend(ctx: *anyopaque) void {
    const self = selfFrom(ctx);
    const allocator = self.allocator;
    const owned = self.owned_by_backend;
    self.deinit();
    if (owned) allocator.destroy(self);
}

/// Best fit out of the pool of released buffers, else a new allocation.
fn allocDeviceBuffer(self: *HipCompute, len: usize) !DeviceBuffer {
    var best: ?usize = null;
    for (self.temp_buffers.items, 0..) |b, i| {
        if (b.len >= len and (best == null or b.len < self.temp_buffers.items[best.?].len)) best = i;
    }
    if (best) |i| return self.temp_buffers.swapRemove(i);
    return DeviceBuffer.alloc(&self.ctx, len);
}

fn releaseDeviceBuffer(self: *HipCompute, buffer: *DeviceBuffer) void {
    if (buffer.ptr == 0) return;
    if (self.temp_buffers.items.len < max_pooled_buffers) {
        self.temp_buffers.append(self.allocator, buffer.*) catch {
            buffer.free(&self.ctx);
            return;
        };
        buffer.* = .{};
    } else {
        // kernels already queued may still read it
        self.ctx.synchronize() catch {};
        buffer.free(&self.ctx);
    }
}

fn freeTensor(ctx: *anyopaque, tensor: CT) void {
    const self = selfFrom(ctx);
    const t = tensorFromCt(tensor);
    if (!t.owned_by_tensor) return; // resident weights are borrowed
    if (t.owns_buffer) releaseDeviceBuffer(self, &t.buffer);
    if (t.owns_shape) self.allocator.free(t.shape);
    self.allocator.destroy(t);
}

fn getWeight(ctx: *anyopaque, name: []const u8) anyerror!CT {
    const self = selfFrom(ctx);
    const entry = self.resident_weights.getPtr(name) orelse return error.WeightNotFound;
    return @ptrCast(entry);
}

fn prefetchWeightHint(_: *anyopaque, _: []const u8, _: u32) void {}
fn drainPrefetchBudget(_: *anyopaque, _: usize) void {}

fn createTensor(self: *HipCompute, device: DeviceBuffer, shape: []i64, elem_count: usize) !CT {
    const t = try self.allocator.create(HipTensor);
    t.* = .{ .buffer = device, .dtype = .f32, .shape = shape, .elem_count = elem_count };
    return @ptrCast(t);
}

fn fromFloat32Op(ctx: *anyopaque, data: []const f32) anyerror!CT {
    const shape = [_]i32{@intCast(data.len)};
    return fromFloat32ShapeOp(ctx, data, &shape);
}

fn fromFloat32ShapeOp(ctx: *anyopaque, data: []const f32, shape: []const i32) anyerror!CT {
    const self = selfFrom(ctx);
    const dims = try self.allocator.alloc(i64, shape.len);
    errdefer self.allocator.free(dims);
    for (shape, dims) |s, *d| d.* = s;
    if (try elementCountFromShape(dims) != data.len) return error.InvalidShape;
    var device = try allocDeviceBuffer(self, data.len * @sizeOf(f32));
    errdefer device.free(&self.ctx);
    try device.copyFromHost(&self.ctx, std.mem.sliceAsBytes(data));
    try self.ctx.synchronize(); // `data` may go away as soon as this returns
    return createTensor(self, device, dims, data.len);
}

fn toFloat32Op(ctx: *anyopaque, tensor: CT, allocator: std.mem.Allocator) anyerror![]f32 {
    const self = selfFrom(ctx);
    const t = tensorFromCt(tensor);
    if (t.dtype != .f32) return error.UnsupportedTensorType;
    const out = try allocator.alloc(f32, t.elem_count);
    errdefer allocator.free(out);
    try t.buffer.copyToHost(&self.ctx, std.mem.sliceAsBytes(out));
    try self.ctx.synchronize();
    return out;
}

fn tensorDTypeOp(_: *anyopaque, tensor: CT) anyerror!tensor_mod.DType {
    return tensorFromCt(tensor).dtype;
}

fn tensorShapeOp(_: *anyopaque, tensor: CT, allocator: std.mem.Allocator) anyerror![]i64 {
    return allocator.dupe(i64, tensorFromCt(tensor).shape);
}

fn evalTensorOp(ctx: *anyopaque, _: CT) anyerror!void {
    try selfFrom(ctx).ctx.synchronize();
}

fn elementCountFromShape(shape: []const i64) !usize {
    var count: usize = 1;
    for (shape) |d| {
        if (d < 0) return error.InvalidShape;
        count = std.math.mul(usize, count, @intCast(d)) catch return error.InvalidShape;
    }
    return count;
}

fn checkedMul(a: usize, b: usize) !usize {
    return std.math.mul(usize, a, b) catch error.InvalidShape;
}

/// ops.zig:890.  X [rows, in_dim] f32, W [out_dim, in_dim] in 32-value blocks along in_dim,
/// Y [rows, out_dim] f32: a new tensor owned by the caller.
fn linearNoBias(ctx: *anyopaque, input: CT, weight: CT, rows: usize, in_dim: usize, out_dim: usize) anyerror!CT {
    const self = selfFrom(ctx);
    const x = tensorFromCt(input);
    const w = tensorFromCt(weight);
    if (x.dtype != .f32) return error.UnsupportedTensorType;
    if (x.elem_count != try checkedMul(rows, in_dim)) return error.InvalidShape;
    if (w.elem_count != try checkedMul(out_dim, in_dim)) return error.InvalidShape;
    const quant = w.quant_type orelse return error.HipOpUnsupported; // dense f32 weights: not this backend's op
    const tt = kernelType(quant) orelse return error.UnsupportedTensorType;
    if (!w.prepared) return error.UnsupportedTensorType;

    const out_count = try checkedMul(rows, out_dim);
    const shape = try self.allocator.alloc(i64, 2);
    errdefer self.allocator.free(shape);
    shape[0] = @intCast(rows);
    shape[1] = @intCast(out_dim);
    var device = try allocDeviceBuffer(self, out_count * @sizeOf(f32));
    errdefer device.free(&self.ctx);
    const workspace = try self.workspace.acquire(&self.ctx, kernels_mod.linearWorkspaceBytes(tt, rows, in_dim, out_dim));
    try self.kernels.launchLinearF32(&self.ctx, tt, device, x.buffer, w.buffer, rows, in_dim, out_dim, workspace);
    return createTensor(self, device, shape, out_count);
}

/// ops.zig:895 with validateQuantLinearPlan (ops/native_compute.zig:5039-5050): the plan has to
/// be a quant_matmul plan for exactly this shape and format.
fn linearNoBiasPlanned(ctx: *anyopaque, request: *const ops.LinearNoBiasPlannedRequest) anyerror!CT {
    const w = tensorFromCt(request.weight);
    const plan = switch (request.operator_plan) {
        .quant_matmul => |p| p,
        else => return error.InvalidPartitionPlan,
    };
    if (plan.rows != request.rows or plan.in_dim != request.in_dim or plan.out_dim != request.out_dim) return error.InvalidPartitionPlan;
    if (w.quant_type == null) return error.UnsupportedOperation;
    _ = operator_plan_mod;
    return linearNoBias(ctx, request.input, request.weight, request.rows, request.in_dim, request.out_dim);
}

// ---- required entries of the op table that are not part of this backend

fn embeddingLookup(_: *anyopaque, _: CT, _: []const i64, _: usize, _: usize) anyerror!CT {
    return error.HipOpUnsupported;
}
fn linear(_: *anyopaque, _: CT, _: CT, _: CT, _: usize, _: usize, _: usize) anyerror!CT {
    return error.HipOpUnsupported;
}
fn layerNorm(_: *anyopaque, _: CT, _: CT, _: CT, _: usize, _: f32) anyerror!CT {
    return error.HipOpUnsupported;
}
fn rmsNorm(_: *anyopaque, _: CT, _: CT, _: usize, _: f32) anyerror!CT {
    return error.HipOpUnsupported;
}
fn unaryUnsupported(_: *anyopaque, _: CT) anyerror!CT {
    return error.HipOpUnsupported;
}
fn binaryUnsupported(_: *anyopaque, _: CT, _: CT) anyerror!CT {
    return error.HipOpUnsupported;
}
fn concat(_: *anyopaque, _: CT, _: CT, _: usize, _: usize, _: usize) anyerror!CT {
    return error.HipOpUnsupported;
}
fn sdpa(_: *anyopaque, _: CT, _: CT, _: CT, _: []const i64, _: ?CT, _: usize, _: usize, _: usize, _: usize) anyerror!CT {
    return error.HipOpUnsupported;
}
fn causalSelfAttention(_: *anyopaque, _: CT, _: CT, _: CT, _: ?CT, _: usize, _: usize, _: usize, _: usize) anyerror!CT {
    return error.HipOpUnsupported;
}
fn crossAttention(_: *anyopaque, _: CT, _: CT, _: CT, _: []const i64, _: usize, _: usize, _: usize, _: usize, _: usize) anyerror!CT {
    return error.HipOpUnsupported;
}
fn relativePositionBias(_: *anyopaque, _: CT, _: usize, _: usize, _: usize, _: usize, _: usize, _: bool) anyerror!CT {
    return error.HipOpUnsupported;
}
fn disentangledRelativeAttention(_: *anyopaque, _: CT, _: CT, _: CT, _: CT, _: CT, _: []const i64, _: usize, _: usize, _: usize, _: usize) anyerror!CT {
    return error.HipOpUnsupported;
}
fn windowedSelfAttention(_: *anyopaque, _: CT, _: CT, _: CT, _: CT, _: CT, _: CT, _: CT, _: usize, _: usize, _: usize, _: usize, _: usize, _: usize) anyerror!CT {
    return error.HipOpUnsupported;
}
fn channelSelfAttention(_: *anyopaque, _: CT, _: CT, _: CT, _: CT, _: CT, _: CT, _: CT, _: usize, _: usize, _: usize, _: usize) anyerror!CT {
    return error.HipOpUnsupported;
}
fn tokenGridConv2d(_: *anyopaque, _: CT, _: CT, _: CT, _: usize, _: usize, _: usize, _: usize, _: usize, _: usize, _: usize, _: usize, _: usize, _: usize, _: usize, _: usize) anyerror!CT {
    return error.HipOpUnsupported;
}
fn conv1d(_: *anyopaque, _: CT, _: CT, _: CT, _: usize, _: usize, _: usize, _: usize, _: usize, _: usize, _: usize) anyerror!CT {
    return error.HipOpUnsupported;
}
fn conv2d(_: *anyopaque, _: CT, _: CT, _: CT, _: usize, _: usize, _: usize, _: usize, _: usize, _: usize, _: usize, _: usize, _: usize, _: usize, _: usize, _: usize) anyerror!CT {
    return error.HipOpUnsupported;
}
fn rope(_: *anyopaque, _: CT, _: usize, _: usize, _: usize, _: f32, _: f32, _: usize, _: bool) anyerror!CT {
    return error.HipOpUnsupported;
}
fn ropePerItem(_: *anyopaque, _: CT, _: usize, _: usize, _: usize, _: usize, _: f32, _: f32, _: []const usize, _: []const usize, _: bool) anyerror!CT {
    return error.HipOpUnsupported;
}
fn gqaCausalAttention(_: *anyopaque, _: CT, _: CT, _: CT, _: ?CT, _: usize, _: usize, _: usize, _: usize, _: usize) anyerror!CT {
    return error.HipOpUnsupported;
}
fn gqaPagedAttention(_: *anyopaque, _: CT, _: CT, _: CT, _: ?CT, _: ops.AttentionContext, _: usize, _: usize, _: usize, _: usize) anyerror!CT {
    return error.HipOpUnsupported;
}

const vtable = ops.ComputeBackend.VTable{
    .backendKind = &backendKind,
    .deinitBackend = &deinitBackend,
    .freeTensor = &freeTensor,
    .getWeight = &getWeight,
    .prefetchWeightHint = &prefetchWeightHint,
    .drainPrefetchBudget = &drainPrefetchBudget,
    .embeddingLookup = &embeddingLookup,
    .linear = &linear,
    .linearNoBias = &linearNoBias,
    .linearNoBiasPlanned = &linearNoBiasPlanned,
    .layerNorm = &layerNorm,
    .rmsNorm = &rmsNorm,
    .gelu = &unaryUnsupported,
    .relu = &unaryUnsupported,
    .silu = &unaryUnsupported,
    .quickGelu = &unaryUnsupported,
    .sigmoid = &unaryUnsupported,
    .tanh_act = &unaryUnsupported,
    .concat = &concat,
    .add = &binaryUnsupported,
    .scaledDotProductAttention = &sdpa,
    .causalSelfAttention = &causalSelfAttention,
    .crossAttention = &crossAttention,
    .relativePositionBias = &relativePositionBias,
    .disentangledRelativeAttention = &disentangledRelativeAttention,
    .windowedSelfAttention = &windowedSelfAttention,
    .channelSelfAttention = &channelSelfAttention,
    .tokenGridConv2d = &tokenGridConv2d,
    .multiply = &binaryUnsupported,
    .conv1d = &conv1d,
    .conv2d = &conv2d,
    .rope = &rope,
    .ropePerItem = &ropePerItem,
    .gqaCausalAttention = &gqaCausalAttention,
    .gqaPagedAttention = &gqaPagedAttention,
    .fromFloat32 = &fromFloat32Op,
    .fromFloat32Shape = &fromFloat32ShapeOp,
    .toFloat32 = &toFloat32Op,
    .tensorDType = &tensorDTypeOp,
    .tensorShape = &tensorShapeOp,
    .evalTensor = &evalTensorOp,
};

test "hip compute op table is type checked" {
    _ = vtable;
}
