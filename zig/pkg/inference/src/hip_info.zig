//! `antfly inference hip-info [--smoke]`: is there a usable HIP device, and do the quantized
//! matmul kernels give the known answers on it (cuda_info.zig:57-82 for the `hip` backend).
const std = @import("std");
const build_options = @import("build_options");

const print = std.debug.print;

const hip_context = if (build_options.enable_hip) @import("ops/hip/context.zig") else struct {};
const hip_kernels = if (build_options.enable_hip) @import("ops/hip/kernels.zig") else struct {};

pub fn main(allocator: std.mem.Allocator, _: std.Io, args: []const []const u8) !void {
    var smoke = false;
    for (args) |arg| {
        if (std.mem.eql(u8, arg, "--smoke")) {
            smoke = true;
        } else if (std.mem.eql(u8, arg, "--help") or std.mem.eql(u8, arg, "-h")) {
            print("usage: antfly inference hip-info [--smoke]\n", .{});
            return;
        } else {
            print("unknown hip-info option: {s}\nusage: antfly inference hip-info [--smoke]\n", .{arg});
            std.process.exit(1);
        }
    }
    if (!build_options.enable_hip) {
        print("hip: unavailable\nreason: backend not built; rebuild with -Dhip=true\n", .{});
        std.process.exit(1);
    }
    if (comptime build_options.enable_hip) {
        const info = hip_context.probeDefault() catch |err| {
            print("hip: unavailable\nreason: {s}\n", .{@errorName(err)});
            std.process.exit(1);
        };
        print("hip: available\ndriver_version: {d}\ndevice_count: {d}\nselected_device: {d}\ndevice_name: {s}\ncompute_units: {d}\n", .{
            info.driver_version, info.device_count, info.selected_device, info.nameSlice(), info.compute_units,
        });
        if (smoke) {
            const Smoke = struct { name: []const u8, run: *const fn (std.mem.Allocator) anyerror!void };
            const smokes = [_]Smoke{
                .{ .name = "q8_0_f32", .run = &hip_kernels.smokeQ8_0 },
                .{ .name = "q4_0_f32", .run = &hip_kernels.smokeQ4_0 },
            };
            for (smokes) |s| {
                s.run(allocator) catch |err| {
                    print("smoke: {s} failed\nreason: {s}\n", .{ s.name, @errorName(err) });
                    std.process.exit(1);
                };
                print("smoke: {s} ok\n", .{s.name});
            }
        }
    }
}
