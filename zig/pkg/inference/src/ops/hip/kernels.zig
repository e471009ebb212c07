//! Kernel module of the `hip` backend: the gfx950 code object, loaded by this backend itself
//! (hipModuleLoadData of the embedded image; ops/cuda/kernels.zig:20-21, :69-218 and
//! :1980-2007 do the same with their image), its entry points, and the launchers the compute
//! ops call (ops/cuda/kernels.zig:1221-1289 for the quantized matmul).
//!
//! Dispatch by rows (graph/quant_matmul.zig:263-268), every bucket from this module's own code object,
//! launched from a parameter block:
//!   small shapes (out_dim < 512 or in_dim < 96)  the f32 route entry (the CPU engine's route gate)
//!   mmv (1 row), small_batch up to 4 rows of Q4_0 / 2 of Q8_0 on K <= 4096
//!                                       the decode entry, activations quantized inside the kernel
//!   small_batch otherwise               the quantizer entry, then the rows entry
//!   mm (9+ rows)                        the quantizer entry, then the int8-MFMA GEMM entry
//! `batch_kernels = .library` (the default) hands 5 .. 128 rows to libantfly_hip_qmatmul's launcher
//! (afhip_launch_linear_f32) instead, whose MFMA batch kernels are faster there; the library is a thin C
//! ABI over the same kernels and owns no device state when called through its afhip_launch_* layer --
//! stream, buffers and module loading stay here.  `.module` keeps every launch in this file.
const std = @import("std");
const buffer_mod = @import("buffer.zig");
const context_mod = @import("context.zig");
const driver_mod = @import("driver.zig");
const quant_matmul = @import("../../graph/quant_matmul.zig");

/// Built by `make -C antfly_amd/csrc` (hipcc --genco --offload-arch=gfx950); normal builds never
/// invoke the device compiler, they embed the prebuilt image.
const code_object = @embedFile("artifacts/antfly_hip_kernels.hsaco");

pub const block_values: usize = 32;
pub const q4_0_block_bytes: usize = 18;
pub const q8_0_block_bytes: usize = 34;

/// GGUF tensor-type ids as the C ABI takes them (gguf/tensor_types.zig).
pub const TensorType = enum(c_int) { q4_0 = 2, q8_0 = 8 };
pub const layout_prepared: c_int = 1;

// ---- C ABI of libantfly_hip_qmatmul.so (include/antfly_hip_qmatmul.h)
pub const AfhipBuffer = buffer_mod.DeviceBuffer; // extern struct { ptr: u64, len: usize }
extern "c" fn afhip_prepared_weight_bytes(tensor_type: c_int, out_dim: usize, in_dim: usize) usize;
extern "c" fn afhip_linear_workspace_bytes(tensor_type: c_int, rows: usize, in_dim: usize, out_dim: usize) usize;
extern "c" fn afhip_launch_linear_f32(
    stream: ?*anyopaque,
    tensor_type: c_int,
    layout: c_int,
    dst: AfhipBuffer,
    input: AfhipBuffer,
    weight: AfhipBuffer,
    rows: usize,
    in_dim: usize,
    out_dim: usize,
    workspace: AfhipBuffer,
    dispatch: c_int,
) c_int;

pub fn preparedWeightBytes(tensor_type: TensorType, out_dim: usize, in_dim: usize) usize {
    return afhip_prepared_weight_bytes(@intFromEnum(tensor_type), out_dim, in_dim);
}

pub fn linearWorkspaceBytes(tensor_type: TensorType, rows: usize, in_dim: usize, out_dim: usize) usize {
    return afhip_linear_workspace_bytes(@intFromEnum(tensor_type), rows, in_dim, out_dim);
}

pub const BatchKernels = enum { module, library };

pub const KernelModule = struct {
    module: driver_mod.hipModule_t = null,
    zero_fill: driver_mod.hipFunction_t = null,
    prepare_weight_q4_0: driver_mod.hipFunction_t = null,
    prepare_weight_q8_0: driver_mod.hipFunction_t = null,
    linear_q4_0_f32: driver_mod.hipFunction_t = null,
    linear_q8_0_f32: driver_mod.hipFunction_t = null,
    linear_q4_0_f32_route: driver_mod.hipFunction_t = null,
    linear_q8_0_f32_route: driver_mod.hipFunction_t = null,
    quantize_activations: driver_mod.hipFunction_t = null,
    linear_q4_0_rows_f32: driver_mod.hipFunction_t = null,
    linear_q8_0_rows_f32: driver_mod.hipFunction_t = null,
    gemm_q4_0_f32: driver_mod.hipFunction_t = null,
    gemm_q8_0_f32: driver_mod.hipFunction_t = null,
    gemm_q4_0_f32_small: driver_mod.hipFunction_t = null,
    gemm_q8_0_f32_small: driver_mod.hipFunction_t = null,
    /// who serves 5 .. 128 rows (see the file comment)
    batch_kernels: BatchKernels = .library,

    pub fn load(ctx: *context_mod.HipContext) driver_mod.Error!KernelModule {
        try ctx.makeCurrent();
        var self = KernelModule{};
        const rc = ctx.driver.fns.hipModuleLoadData(&self.module, code_object.ptr);
        if (rc != driver_mod.hipSuccess) {
            std.debug.print("hip: code object load failed: {s}: {s}\n", .{ ctx.driver.errorName(rc), ctx.driver.errorString(rc) });
            return error.HipDriverError;
        }
        errdefer _ = ctx.driver.fns.hipModuleUnload(self.module);
        const entries = .{
            .{ &self.zero_fill, "termite_hip_zero_fill" },
            .{ &self.prepare_weight_q4_0, "termite_hip_prepare_weight_q4_0" },
            .{ &self.prepare_weight_q8_0, "termite_hip_prepare_weight_q8_0" },
            .{ &self.linear_q4_0_f32, "termite_hip_linear_q4_0_f32" },
            .{ &self.linear_q8_0_f32, "termite_hip_linear_q8_0_f32" },
            .{ &self.linear_q4_0_f32_route, "termite_hip_linear_q4_0_f32_route" },
            .{ &self.linear_q8_0_f32_route, "termite_hip_linear_q8_0_f32_route" },
            .{ &self.quantize_activations, "termite_hip_quantize_activations" },
            .{ &self.linear_q4_0_rows_f32, "termite_hip_linear_q4_0_rows_f32" },
            .{ &self.linear_q8_0_rows_f32, "termite_hip_linear_q8_0_rows_f32" },
            .{ &self.gemm_q4_0_f32, "termite_hip_gemm_q4_0_f32" },
            .{ &self.gemm_q8_0_f32, "termite_hip_gemm_q8_0_f32" },
            .{ &self.gemm_q4_0_f32_small, "termite_hip_gemm_q4_0_f32_small" },
            .{ &self.gemm_q8_0_f32_small, "termite_hip_gemm_q8_0_f32_small" },
        };
        inline for (entries) |entry| {
            try ctx.driver.check(ctx.driver.fns.hipModuleGetFunction(entry[0], self.module, entry[1]));
        }
        return self;
    }

    pub fn unload(self: *KernelModule, ctx: *context_mod.HipContext) void {
        if (self.module == null) return;
        ctx.makeCurrent() catch {};
        _ = ctx.driver.fns.hipModuleUnload(self.module);
        self.* = .{};
    }

    /// RAW GGUF blocks -> the PREPARED layout the kernels read (quant bytes, fp16 scales in block
    /// order, the scales once more in wavefront-tile order).  One-time, at weight load.
    pub fn launchPrepareWeight(
        self: *KernelModule,
        ctx: *context_mod.HipContext,
        tensor_type: TensorType,
        dst_prepared: buffer_mod.DeviceBuffer,
        src_raw: buffer_mod.DeviceBuffer,
        out_dim: usize,
        in_dim: usize,
    ) driver_mod.Error!void {
        if (in_dim == 0 or in_dim % block_values != 0) return error.InvalidHipState;
        const kb = in_dim / block_values;
        const raw_block: usize = if (tensor_type == .q4_0) q4_0_block_bytes else q8_0_block_bytes;
        const blocks = try checkedMul(out_dim, kb);
        const raw_bytes = try checkedMul(blocks, raw_block);
        const prepared = preparedWeightBytes(tensor_type, out_dim, in_dim);
        if (raw_bytes > src_raw.len or prepared == 0 or prepared > dst_prepared.len) return error.InvalidHipState;
        if (blocks == 0) return;
        // zero from the 16-byte unit that holds the end of the block-order scales to the end
        const fill_from = raw_bytes & ~@as(usize, 15);
        var fill_ptr: u64 = dst_prepared.ptr + fill_from;
        var fill_n16: u64 = (prepared - fill_from) / 16;
        var fill_params = [_]?*anyopaque{ @ptrCast(&fill_ptr), @ptrCast(&fill_n16) };
        try launch(ctx, self.zero_fill, .{ gridFor(fill_n16, 256, 4096), 1 }, .{ 256, 1 }, 0, &fill_params);

        var dst_ptr = dst_prepared.ptr;
        var src_ptr = src_raw.ptr;
        var out_u32 = try toU32(out_dim);
        var kb_u32 = try toU32(kb);
        var params = [_]?*anyopaque{ @ptrCast(&dst_ptr), @ptrCast(&src_ptr), @ptrCast(&out_u32), @ptrCast(&kb_u32) };
        const f = if (tensor_type == .q4_0) self.prepare_weight_q4_0 else self.prepare_weight_q8_0;
        try launch(ctx, f, .{ gridFor(blocks, 256, std.math.maxInt(u32)), 1 }, .{ 256, 1 }, 0, &params);
    }

    /// Y[rows, out_dim] = X[rows, in_dim] * W^T for a PREPARED Q4_0 / Q8_0 weight.  Same argument
    /// checks as ops/cuda/kernels.zig:1231-1236; `workspace` must hold linearWorkspaceBytes().
    pub fn launchLinearF32(
        self: *KernelModule,
        ctx: *context_mod.HipContext,
        tensor_type: TensorType,
        dst: buffer_mod.DeviceBuffer,
        input: buffer_mod.DeviceBuffer,
        weight_prepared: buffer_mod.DeviceBuffer,
        rows: usize,
        in_dim: usize,
        out_dim: usize,
        workspace: buffer_mod.DeviceBuffer,
    ) driver_mod.Error!void {
        if (in_dim == 0 or in_dim % block_values != 0) return error.InvalidHipState;
        const out_count = try checkedMul(rows, out_dim);
        try checkBytes(dst, try checkedMul(out_count, @sizeOf(f32)));
        try checkBytes(input, try checkedMul(try checkedMul(rows, in_dim), @sizeOf(f32)));
        try checkBytes(weight_prepared, preparedWeightBytes(tensor_type, out_dim, in_dim));
        if (out_count == 0) return;

        const format: quant_matmul.Format = if (tensor_type == .q4_0) .q4_0 else .q8_0;
        const kind = quant_matmul.select(.{ .rows = rows, .in_dim = in_dim, .out_dim = out_dim, .format = format });
        const kb = in_dim / block_values;
        // the CPU engine's route gate (ops/native_compute.zig:3410-3419): small shapes multiply f32
        // activations by dequantized weights
        const activation_quant = out_dim >= 512 and kb >= 3;
        if (!activation_quant) return self.launchF32Route(ctx, tensor_type, dst, input, weight_prepared, rows, in_dim, out_dim);
        // activations quantized inside the decode kernel: one row up to K = 16384; up to 4 (Q4_0) / 2 (Q8_0)
        // rows on one K slice, at most 512 blocks of X from three rows on
        const fused_rows: usize = if (tensor_type == .q4_0) 4 else 2;
        const fused = (rows == 1 and kb <= 16 * 128) or
            (rows >= 2 and rows <= fused_rows and kb <= 128 and (rows <= 2 or rows * kb <= 512));
        if (kind != .mm and fused) {
            return self.launchDecodeRows(ctx, tensor_type, dst, input, weight_prepared, rows, in_dim, out_dim);
        }
        if (self.batch_kernels == .library and rows >= 5 and rows <= 128) {
            try ctx.makeCurrent();
            const rc = afhip_launch_linear_f32(ctx.stream, @intFromEnum(tensor_type), layout_prepared, dst, input, weight_prepared, rows, in_dim, out_dim, workspace, -1);
            if (rc != 0) return error.HipDriverError;
            return;
        }
        // quantized activations in the workspace: int8 [rows][in_dim], then f32 scales and i32 sums [rows][kb]
        const q_bytes = try checkedMul(rows, in_dim);
        const s_bytes = try checkedMul(try checkedMul(rows, kb), @sizeOf(f32));
        if (workspace.ptr % 16 != 0 or q_bytes % 16 != 0) return error.InvalidHipState;
        try checkBytes(workspace, q_bytes + 2 * s_bytes);
        const q = buffer_mod.DeviceBuffer{ .ptr = workspace.ptr, .len = q_bytes };
        const scales = buffer_mod.DeviceBuffer{ .ptr = workspace.ptr + q_bytes, .len = s_bytes };
        const sums = buffer_mod.DeviceBuffer{ .ptr = workspace.ptr + q_bytes + s_bytes, .len = s_bytes };
        try self.launchQuantizeActivations(ctx, q, scales, sums, input, rows, in_dim);
        if (kind == .mm) {
            return self.launchGemm(ctx, tensor_type, dst, input, weight_prepared, rows, in_dim, out_dim, q, scales);
        }
        return self.launchRows(ctx, tensor_type, dst, input, weight_prepared, rows, in_dim, out_dim, q, scales, sums);
    }

    /// Route B: grid (out_dim, rows), one wavefront per output element.
    fn launchF32Route(
        self: *KernelModule,
        ctx: *context_mod.HipContext,
        tensor_type: TensorType,
        dst: buffer_mod.DeviceBuffer,
        input: buffer_mod.DeviceBuffer,
        weight_prepared: buffer_mod.DeviceBuffer,
        rows: usize,
        in_dim: usize,
        out_dim: usize,
    ) driver_mod.Error!void {
        var dst_ptr = dst.ptr;
        var input_ptr = input.ptr;
        var weight_ptr = weight_prepared.ptr;
        var rows_u32 = try toU32(rows);
        var in_dim_u32 = try toU32(in_dim);
        var out_dim_u32 = try toU32(out_dim);
        var params = [_]?*anyopaque{ @ptrCast(&dst_ptr), @ptrCast(&input_ptr), @ptrCast(&weight_ptr), @ptrCast(&rows_u32), @ptrCast(&in_dim_u32), @ptrCast(&out_dim_u32) };
        const f = if (tensor_type == .q4_0) self.linear_q4_0_f32_route else self.linear_q8_0_f32_route;
        if (rows > 65535) return error.InvalidHipState; // grid.y
        try launch(ctx, f, .{ try toU32(out_dim), try toU32(rows) }, .{ 64, 1 }, 0, &params);
    }

    /// int8 values, f32 scales and i32 sums of every 32-value block of X (ops/native_compute.zig:23799-23832).
    fn launchQuantizeActivations(
        self: *KernelModule,
        ctx: *context_mod.HipContext,
        q: buffer_mod.DeviceBuffer,
        scales: buffer_mod.DeviceBuffer,
        sums: buffer_mod.DeviceBuffer,
        input: buffer_mod.DeviceBuffer,
        rows: usize,
        in_dim: usize,
    ) driver_mod.Error!void {
        var q_ptr = q.ptr;
        var scales_ptr = scales.ptr;
        var sums_ptr = sums.ptr;
        var input_ptr = input.ptr;
        var rows_u32 = try toU32(rows);
        var in_dim_u32 = try toU32(in_dim);
        var params = [_]?*anyopaque{ @ptrCast(&q_ptr), @ptrCast(&scales_ptr), @ptrCast(&sums_ptr), @ptrCast(&input_ptr), @ptrCast(&rows_u32), @ptrCast(&in_dim_u32) };
        const units: u64 = @intCast(try checkedMul(rows, in_dim / 4));
        try launch(ctx, self.quantize_activations, .{ gridFor(units, 256, 4096), 1 }, .{ 256, 1 }, 0, &params);
    }

    /// small_batch from quantized activations: eight wavefronts a workgroup (a multiple of the K slices).
    fn launchRows(
        self: *KernelModule,
        ctx: *context_mod.HipContext,
        tensor_type: TensorType,
        dst: buffer_mod.DeviceBuffer,
        input: buffer_mod.DeviceBuffer,
        weight_prepared: buffer_mod.DeviceBuffer,
        rows: usize,
        in_dim: usize,
        out_dim: usize,
        q: buffer_mod.DeviceBuffer,
        scales: buffer_mod.DeviceBuffer,
        sums: buffer_mod.DeviceBuffer,
    ) driver_mod.Error!void {
        const kb = in_dim / block_values;
        const cols: usize = if (tensor_type == .q4_0) 4 else 2;
        const slices = (kb + 127) / 128;
        if (slices > 16) return error.InvalidHipState;
        const waves = @max(8 / slices * slices, slices);
        const groups = (out_dim + cols - 1) / cols;
        const groups_per_wg = waves / slices;
        const grid = (groups + groups_per_wg - 1) / groups_per_wg;
        const lds = fusedLdsBytes(rows, in_dim);
        if (lds > 160 * 1024) return error.InvalidHipState; // more rows than LDS holds: the caller slices them
        var dst_ptr = dst.ptr;
        var input_ptr = input.ptr;
        var weight_ptr = weight_prepared.ptr;
        var rows_u32 = try toU32(rows);
        var in_dim_u32 = try toU32(in_dim);
        var out_dim_u32 = try toU32(out_dim);
        var q_ptr = q.ptr;
        var scales_ptr = scales.ptr;
        var sums_ptr = sums.ptr;
        var params = [_]?*anyopaque{ @ptrCast(&dst_ptr), @ptrCast(&input_ptr), @ptrCast(&weight_ptr), @ptrCast(&rows_u32), @ptrCast(&in_dim_u32), @ptrCast(&out_dim_u32), @ptrCast(&q_ptr), @ptrCast(&scales_ptr), @ptrCast(&sums_ptr) };
        const f = if (tensor_type == .q4_0) self.linear_q4_0_rows_f32 else self.linear_q8_0_rows_f32;
        try launch(ctx, f, .{ try toU32(grid), 1 }, .{ try toU32(64 * waves), 1 }, try toU32(lds), &params);
    }

    /// The mm bucket: 64 x 128 tiles while they give every compute unit a workgroup, 32 x 64 tiles otherwise.
    fn launchGemm(
        self: *KernelModule,
        ctx: *context_mod.HipContext,
        tensor_type: TensorType,
        dst: buffer_mod.DeviceBuffer,
        input: buffer_mod.DeviceBuffer,
        weight_prepared: buffer_mod.DeviceBuffer,
        rows: usize,
        in_dim: usize,
        out_dim: usize,
        q: buffer_mod.DeviceBuffer,
        scales: buffer_mod.DeviceBuffer,
    ) driver_mod.Error!void {
        const units: usize = @intCast(@max(ctx.info.compute_units, 1));
        const big = ((rows + 63) / 64) * ((out_dim + 127) / 128) >= units;
        const tile_m: usize = if (big) 64 else 32;
        const tile_n: usize = if (big) 128 else 64;
        const m_tiles = (rows + tile_m - 1) / tile_m;
        const n_tiles = (out_dim + tile_n - 1) / tile_n;
        const grid = try checkedMul(try checkedMul((n_tiles + 7) / 8, m_tiles), 8);
        // four stages of operands: 27648 bytes each, and 8192 more for Q4_0's nibble chunks
        const lds: usize = if (tensor_type == .q4_0) 143360 else 110592;
        var dst_ptr = dst.ptr;
        var input_ptr = input.ptr;
        var weight_ptr = weight_prepared.ptr;
        var rows_u32 = try toU32(rows);
        var in_dim_u32 = try toU32(in_dim);
        var out_dim_u32 = try toU32(out_dim);
        var q_ptr = q.ptr;
        var scales_ptr = scales.ptr;
        var m_tiles_u32 = try toU32(m_tiles);
        var n_tiles_u32 = try toU32(n_tiles);
        var params = [_]?*anyopaque{ @ptrCast(&dst_ptr), @ptrCast(&input_ptr), @ptrCast(&weight_ptr), @ptrCast(&rows_u32), @ptrCast(&in_dim_u32), @ptrCast(&out_dim_u32), @ptrCast(&q_ptr), @ptrCast(&scales_ptr), @ptrCast(&m_tiles_u32), @ptrCast(&n_tiles_u32) };
        const f = if (tensor_type == .q4_0)
            (if (big) self.gemm_q4_0_f32 else self.gemm_q4_0_f32_small)
        else
            (if (big) self.gemm_q8_0_f32 else self.gemm_q8_0_f32_small);
        const threads: u32 = if (big) 1024 else 512;
        try launch(ctx, f, .{ try toU32(grid), 1 }, .{ threads, 1 }, try toU32(lds), &params);
    }

    /// The mmv bucket and the first rows of small_batch: launched from a parameter block whose leading
    /// entries are the reference kernel's (dst, input, weight, rows, in_dim, out_dim).
    fn launchDecodeRows(
        self: *KernelModule,
        ctx: *context_mod.HipContext,
        tensor_type: TensorType,
        dst: buffer_mod.DeviceBuffer,
        input: buffer_mod.DeviceBuffer,
        weight_prepared: buffer_mod.DeviceBuffer,
        rows: usize,
        in_dim: usize,
        out_dim: usize,
    ) driver_mod.Error!void {
        const kb = in_dim / block_values;
        const cols: usize = if (tensor_type == .q4_0) 4 else 2; // output columns per wavefront
        const slices = (kb + 127) / 128; // wavefronts that share one column group along K
        const groups = (out_dim + cols - 1) / cols;
        const units: usize = @intCast(@max(ctx.info.compute_units, 1));
        const groups_per_wg = decodeGroupsPerWorkgroup(groups, slices, units, (rows * kb + 127) / 128);
        const grid = (groups + groups_per_wg - 1) / groups_per_wg;

        var dst_ptr = dst.ptr;
        var input_ptr = input.ptr;
        var weight_ptr = weight_prepared.ptr;
        var rows_u32 = try toU32(rows);
        var in_dim_u32 = try toU32(in_dim);
        var out_dim_u32 = try toU32(out_dim);
        var groups_u32 = try toU32(groups_per_wg);
        var stagger_u32: u32 = if (grid <= units) 1 else 0;
        var params = [_]?*anyopaque{
            @ptrCast(&dst_ptr),
            @ptrCast(&input_ptr),
            @ptrCast(&weight_ptr),
            @ptrCast(&rows_u32),
            @ptrCast(&in_dim_u32),
            @ptrCast(&out_dim_u32),
            @ptrCast(&groups_u32),
            @ptrCast(&stagger_u32),
        };
        const lds = fusedLdsBytes(rows, in_dim);
        const f = if (tensor_type == .q4_0) self.linear_q4_0_f32 else self.linear_q8_0_f32;
        try launch(ctx, f, .{ try toU32(grid), 1 }, .{ try toU32(64 * slices), try toU32(groups_per_wg) }, try toU32(lds), &params);
    }
};

/// Column groups per workgroup for the decode kernel: at most 16 wavefronts per workgroup, and
/// among the sizes that need the fewest rounds of workgroups over the compute units the one
/// with the least streaming + prologue work per unit (every workgroup quantizes X once).
fn decodeGroupsPerWorkgroup(groups: usize, slices: usize, units: usize, x_waves_min: usize) usize {
    const max_groups = @max(16 / slices, 1);
    const min_groups = @max((@max(x_waves_min, 2) + slices - 1) / slices, 1);
    var best = max_groups;
    var best_cost: usize = std.math.maxInt(usize);
    var g = max_groups;
    while (g >= min_groups and g >= 1) : (g -= 1) {
        const grid = (groups + g - 1) / g;
        const cost = ((grid + units - 1) / units) * (g * slices + 2);
        if (cost < best_cost) {
            best_cost = cost;
            best = g;
        }
        if (g == 1) break;
    }
    return best;
}

/// LDS of the decode and rows entries: quantized X (int8 + f32 scale + i32 sum per block) and one partial-sum
/// slot per wavefront, row and column.
fn fusedLdsBytes(rows: usize, in_dim: usize) usize {
    return rows * (in_dim + in_dim / block_values * 8) + 256 * @max(rows, 4);
}

fn launch(
    ctx: *context_mod.HipContext,
    f: driver_mod.hipFunction_t,
    grid: [2]u32,
    block: [2]u32,
    shared_bytes: u32,
    params: []?*anyopaque,
) driver_mod.Error!void {
    if (f == null) return error.InvalidHipState;
    try ctx.makeCurrent();
    try ctx.driver.check(ctx.driver.fns.hipModuleLaunchKernel(f, grid[0], grid[1], 1, block[0], block[1], 1, shared_bytes, ctx.stream, params.ptr, null));
}

fn gridFor(units: u64, per_block: u64, cap: u64) u32 {
    const blocks = @max((units + per_block - 1) / per_block, 1);
    return @intCast(@min(blocks, cap));
}

fn checkedMul(a: usize, b: usize) driver_mod.Error!usize {
    return std.math.mul(usize, a, b) catch error.InvalidHipState;
}

fn checkBytes(buffer: buffer_mod.DeviceBuffer, bytes: usize) driver_mod.Error!void {
    if (bytes > buffer.len) return error.InvalidHipState;
}

fn toU32(value: usize) driver_mod.Error!u32 {
    return std.math.cast(u32, value) orelse error.InvalidHipState;
}

// ---- known-answer smokes (what `hip-info --smoke` runs): the reference's own vectors,
// ops/cuda/kernels.zig:2309-2399 -- X = [1..32; -1..-32], three weight rows (scale, value) =
// (1.0, 1), (0.5, 2), (2.0, -1), expected {528, 528, -1056, -528, -528, 1056}.

fn smokeRow(tensor_type: TensorType, out: []u8, scale_bits: u16, value: i8) void {
    out[0] = @truncate(scale_bits);
    out[1] = @truncate(scale_bits >> 8);
    if (tensor_type == .q8_0) {
        @memset(out[2..34], @bitCast(value));
    } else {
        const nibble: u8 = @intCast(@as(i16, value) + 8);
        @memset(out[2..18], nibble | (nibble << 4));
    }
}

fn smokeLinear(tensor_type: TensorType) !void {
    var ctx = try context_mod.HipContext.initDefault();
    defer ctx.deinit();
    var module = try KernelModule.load(&ctx);
    defer module.unload(&ctx);

    const rows = 2;
    const in_dim = 32;
    const out_dim = 3;
    var x: [rows * in_dim]f32 = undefined;
    for (0..in_dim) |i| {
        x[i] = @floatFromInt(i + 1);
        x[in_dim + i] = -@as(f32, @floatFromInt(i + 1));
    }
    const block: usize = if (tensor_type == .q4_0) q4_0_block_bytes else q8_0_block_bytes;
    var raw: [3 * q8_0_block_bytes]u8 = .{0} ** (3 * q8_0_block_bytes);
    smokeRow(tensor_type, raw[0 * block ..], 0x3C00, 1);
    smokeRow(tensor_type, raw[1 * block ..], 0x3800, 2);
    smokeRow(tensor_type, raw[2 * block ..], 0x4000, -1);

    var raw_dev = try buffer_mod.DeviceBuffer.alloc(&ctx, out_dim * block);
    defer raw_dev.free(&ctx);
    var prepared = try buffer_mod.DeviceBuffer.alloc(&ctx, preparedWeightBytes(tensor_type, out_dim, in_dim));
    defer prepared.free(&ctx);
    var x_dev = try buffer_mod.DeviceBuffer.alloc(&ctx, @sizeOf(@TypeOf(x)));
    defer x_dev.free(&ctx);
    var y_dev = try buffer_mod.DeviceBuffer.alloc(&ctx, rows * out_dim * @sizeOf(f32));
    defer y_dev.free(&ctx);
    var scratch = try buffer_mod.DeviceBuffer.alloc(&ctx, @max(linearWorkspaceBytes(tensor_type, rows, in_dim, out_dim), 16));
    defer scratch.free(&ctx);

    try raw_dev.copyFromHost(&ctx, raw[0 .. out_dim * block]);
    try x_dev.copyFromHost(&ctx, std.mem.sliceAsBytes(x[0..]));
    try module.launchPrepareWeight(&ctx, tensor_type, prepared, raw_dev, out_dim, in_dim);
    try module.launchLinearF32(&ctx, tensor_type, y_dev, x_dev, prepared, rows, in_dim, out_dim, scratch);
    var y: [rows * out_dim]f32 = undefined;
    try y_dev.copyToHost(&ctx, std.mem.sliceAsBytes(y[0..]));
    try ctx.synchronize();

    const expected = [_]f32{ 528, 528, -1056, -528, -528, 1056 };
    for (expected, y) |want, got| {
        if (@abs(got - want) > 0.01) return error.HipSmokeMismatch;
    }
}

pub fn smokeQ8_0(_: std.mem.Allocator) !void {
    try smokeLinear(.q8_0);
}

pub fn smokeQ4_0(_: std.mem.Allocator) !void {
    try smokeLinear(.q4_0);
}

test "decode launch geometry spreads the FFN-up matrix one workgroup per compute unit" {
    // 14336 columns, K = 4096: 3584 column groups, one slice; 14 wavefronts x 256 workgroups
    try std.testing.expectEqual(@as(usize, 14), decodeGroupsPerWorkgroup(3584, 1, 256, 1));
    // K = 14336: four slices per column group, four groups per 16-wavefront workgroup
    try std.testing.expectEqual(@as(usize, 4), decodeGroupsPerWorkgroup(1024, 4, 256, 4));
}
