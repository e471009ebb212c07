//! `--backend hip`: a session whose resident quantized weights live on the MI355X and whose
//! quantized `linearNoBias` runs there (session_factory.zig:1261-1301 builds the CUDA session
//! the same way).  session_factory.zig imports this file behind `build_options.enable_hip`, re-exports
//! `createHipSession*`, adds `hip: HipData` to its `BackendData` and the `hip` arms to its switches:
//! zig/patches/0009 holds that edit as a diff, 0001 .. 0010 the rest of the wiring from `-Dhip` and
//! `--backend hip` down to here.
const std = @import("std");
const build_options = @import("build_options");
const factory = @import("session_factory.zig");
const hip_compute_mod = @import("../ops/hip/hip_compute.zig");

const Session = factory.Session;
const ArchSession = factory.ArchSession;
const TaskOverride = factory.TaskOverride;

pub fn createHipSession(allocator: std.mem.Allocator, model_path: []const u8) !Session {
    return createHipSessionWithTaskOverride(allocator, model_path, null);
}

pub fn createHipSessionWithTaskOverride(allocator: std.mem.Allocator, model_path: []const u8, override: ?TaskOverride) !Session {
    if (comptime !build_options.enable_hip) return error.HipNotEnabled;

    // the native loader reads the GGUF file and keeps quantized tensors as raw bytes
    var native_session = try factory.createNativeSessionWithTaskOverride(allocator, model_path, override);
    defer native_session.close();
    const native_impl: *ArchSession = @ptrCast(@alignCast(native_session.ptr));
    if (native_impl.backend_type != .native) return error.InvalidBackend;

    var hip_compute = try hip_compute_mod.HipCompute.init(allocator);
    errdefer hip_compute.deinit();
    var it = native_impl.backend_data.native.resident_weights.iterator();
    while (it.next()) |entry| {
        if (entry.value_ptr.quantized_storage == null) continue; // dense tensors stay with the host ops
        const owned_key = try allocator.dupe(u8, entry.key_ptr.*);
        hip_compute.insertWeightFromLoaded(owned_key, entry.value_ptr) catch |err| {
            allocator.free(owned_key);
            return err;
        };
    }

    const impl = try allocator.create(ArchSession);
    impl.* = .{
        .allocator = allocator,
        .arch_config = native_impl.arch_config,
        .task = native_impl.task,
        .backend_type = .hip,
        .backend_data = .{ .hip = .{ .compute = hip_compute } },
    };
    return .{ .ptr = impl, .vtable = factory.archVTable() };
}
