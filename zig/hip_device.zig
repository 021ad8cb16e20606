//! HipDevice: Zigrad's second device, backed by libzg_hip.so (include/zg_hip.h).
//!
//! Drop this file into src/device/ next to host_device.zig, add a `hip: *HipDevice` field to the device union in
//! enabled_devices.zig (next to the cuda entry), link libzg_hip.so, and every NDArray / NDTensor / Graph / nn
//! call that goes through DeviceReference.dispatch runs on the MI355X unchanged.
//!
//! The struct follows the reference's duck-typed device contract (src/device/device_reference.zig:15-131):
//! one method per opspec `__name__` with the signature `fn (self, T: type, p: opspec.<name>(T)) void`, the
//! mem_* API, `reference()`, `sync()`.  Ops cannot return errors in that contract, so a non-zero return
//! code from the C ABI becomes @panic with the library's message, as the CUDA C layer exits on error
//! (src/cuda/cuda_helpers.cu:21-28).
//!
//! This file cannot be compiled in the build container (no Zig toolchain); it is written against Zig 0.14
//! and the reference's tree layout; the reference's own device-parameterised tests (tests/src/main.zig:21-27)
//! are what exercises it.
const std = @import("std");
const c = @cImport(@cInclude("zg_hip.h"));
const opspec = @import("opspec.zig");
const RandType = @import("device_common.zig").RandType;
const TransferDirection = @import("device_common.zig").TransferDirection;
const allocators = @import("../allocators.zig");
const DeviceData = allocators.DeviceData;
const Error = allocators.Error;
const adjust_map_size = allocators.adjust_map_size;

pub const DeviceReference = @import("device_reference.zig");
const Self = @This();

fn check(rc: c_int) void {
    if (rc != 0) std.debug.panic("zg_hip: {s}", .{std.mem.span(c.zg_hip_last_error())});
}

/// The per-device handler src/allocators/caching_allocator.zig is generic over, for a build that wants Zigrad's own
/// `CachingAllocator(HipDevice.DataHandler)` over device memory (every member the contract names:
/// src/allocators/block_pool.zig:103-173).  `map` hands the block pool one contiguous device region; `map_alloc` is
/// left out on purpose (src/allocators/block_pool.zig:115 makes it optional): the region is physically backed when
/// mapped.  The device below does NOT use it: its mem_cache_* methods go through the library's allocator
/// (zg_hip_mem_cache_*), the one the library's tests cover and the one that knows about execution graphs.
pub const DataHandler = struct {
    pub const min_split_size = 256; // bytes; every block is then 256-byte aligned, enough for 128-bit accesses

    ctx: *c.zg_hip_ctx,

    pub fn map(self: DataHandler, size: ?usize) Error![]u8 {
        var total: usize = 0;
        check(c.zg_hip_total_memory(self.ctx, &total));
        // default: a quarter of the device per pool instead of over-subscribing all of it
        const want = adjust_map_size(size orelse total / 4, self.page_size(), total);
        var ptr: ?*anyopaque = null;
        if (c.zg_hip_pool_map(self.ctx, want, &ptr) != 0) return Error.DeviceOOM;
        const bytes: [*]u8 = @ptrCast(ptr.?);
        return bytes[0..want];
    }
    pub fn unmap(self: DataHandler, buf: []u8) void {
        check(c.zg_hip_pool_unmap(self.ctx, buf.ptr));
    }
    pub fn alloc(self: DataHandler, n: usize) ?[*]u8 {
        var ptr: ?*anyopaque = null;
        if (c.zg_hip_alloc(self.ctx, n, &ptr) != 0) return null;
        return @ptrCast(ptr.?);
    }
    pub fn free(self: DataHandler, buf: []u8) void {
        check(c.zg_hip_free(self.ctx, buf.ptr));
    }
    pub fn page_size(self: DataHandler) usize {
        var n: usize = 0;
        check(c.zg_hip_page_size(self.ctx, &n));
        return n;
    }
    pub inline fn reset(_: DataHandler) void {}
    pub fn deinit(self: *DataHandler) void {
        self.* = undefined;
    }
};

/// Segment sizes of the library's two block pools (the counterpart of CachingAllocator.Options,
/// src/allocators/caching_allocator.zig:41-44); null keeps the library's defaults (64 MiB and 1 GiB).
pub const Options = struct {
    small_pool_size: ?usize = null,
    large_pool_size: ?usize = null,
};

ctx: *c.zg_hip_ctx,

pub fn device_count() u32 {
    var n: c_int = 0;
    check(c.zg_hip_device_count(&n));
    return @intCast(n);
}

pub fn init(device_number: u32) Self {
    return init_advanced(device_number, .{});
}

pub fn init_advanced(device_number: u32, opts: Options) Self {
    var ctx: ?*c.zg_hip_ctx = null;
    check(c.zg_hip_init(@intCast(device_number), &ctx));
    if (opts.small_pool_size != null or opts.large_pool_size != null)
        check(c.zg_hip_cache_configure(ctx.?, opts.small_pool_size orelse (64 << 20), opts.large_pool_size orelse (1 << 30)));
    return .{ .ctx = ctx.? };
}

pub fn deinit(self: *Self) void {
    self.sync();
    check(c.zg_hip_deinit(self.ctx)); // frees the pools, the scratch buffer and every raw allocation still live
    self.* = undefined;
}

pub fn reference(self: *Self) DeviceReference {
    return .{ .ptrs = .{ .hip = self } };
}

pub fn is_compatible(self: *const Self, other: *const Self) bool {
    return self.ctx == other.ctx;
}

pub fn sync(self: *const Self) void {
    check(c.zg_hip_sync(self.ctx));
}

pub fn clear_cache(self: *Self) void {
    check(c.zg_hip_clear_cache(self.ctx));
}

// --------------------------------------------------------------------------------------------------
// Host-pointer hazards.  Callers that grew up on the host device touch host memory in three places, and none of
// them has to change:
//   - the scalar operand of add_scalar & co is a one-element slice on the caller's stack (src/ndarray.zig:247-257):
//     `binary` below passes it BY VALUE (zg_hip_add_scalar ...), so nothing is copied or waited for;
//   - axpy's alpha (src/nn/optim.zig:117) is read on the host at call time (`axpy` below);
//   - `usize` buffers are read and written through `.raw` by host loops (NDArray.gather, src/ndarray.zig:607-624;
//     the GCN's edge lists, examples/gcn/src/model.zig:204-205): every allocation of `usize` elements, cached or
//     not, is pinned host memory that the kernels read in place, and every device op that writes one is followed
//     by a wait, so the host loops see what HostDevice would show them.
// --------------------------------------------------------------------------------------------------
fn is_device_ptr(self: *const Self, p: *const anyopaque) bool {
    var yes: c_int = 0;
    check(c.zg_hip_is_device_ptr(self.ctx, p, &yes)); // a host-side range test; launches nothing, flushes nothing
    return yes != 0;
}

/// DeviceData.ctx of a cached `usize` allocation: pinned host memory, not a block of the device pools.
const host_tag: usize = std.math.maxInt(usize);

fn host_alloc(self: *const Self, T: type, n: usize) ![]T {
    var ptr: ?*anyopaque = null;
    if (c.zg_hip_host_alloc(self.ctx, n * @sizeOf(T), &ptr) != 0) return Error.DeviceOOM;
    const p: [*]T = @ptrCast(@alignCast(ptr.?));
    return p[0..n];
}

/// Kept for callers that ask for index memory by name; `mem_alloc(usize, n)` returns the same kind of memory.
pub fn mem_alloc_indices(self: *Self, n: usize) ![]usize {
    return self.host_alloc(usize, n);
}

// --------------------------------------------------------------------------------------------------
// memory API (src/device/device_reference.zig:29-123)
// --------------------------------------------------------------------------------------------------
/// `ctx` of the returned DeviceData is the library's block handle (the reference keeps its *Block there:
/// src/allocators/device_data.zig:32-40, src/allocators/block_pool.zig:262-269); views carry 0 and are never freed.
pub fn mem_cache_alloc(self: *Self, T: type, n: usize) !DeviceData(T) {
    if (n == 0) return .{ .raw = &.{}, .ctx = 0 }; // src/allocators/caching_allocator.zig:81-85
    if (T == usize) return .{ .raw = try self.host_alloc(T, n), .ctx = host_tag }; // host loops read and write it
    var ptr: ?*anyopaque = null;
    var block: u64 = 0;
    if (c.zg_hip_mem_cache_alloc(self.ctx, n * @sizeOf(T), &ptr, &block) != 0) return Error.DeviceOOM;
    const p: [*]T = @ptrCast(@alignCast(ptr.?));
    return .{ .raw = p[0..n], .ctx = @intCast(block) };
}
pub fn mem_cache_free(self: *Self, data: anytype) void {
    if (data.raw.len == 0 or data.ctx == 0) return; // src/allocators/caching_allocator.zig:111-112
    if (data.ctx == host_tag) return check(c.zg_hip_host_free(self.ctx, @constCast(@ptrCast(data.raw.ptr))));
    check(c.zg_hip_mem_cache_free(self.ctx, @constCast(@ptrCast(data.raw.ptr)), @intCast(data.ctx)));
}
pub fn mem_cache_dupe(self: *Self, T: type, src: []const T) !DeviceData(T) {
    const dst = try self.mem_cache_alloc(T, src.len);
    // callers pass host stack values here (src/nn/loss.zig:163), so pick the direction by where src lives
    if (self.is_device_ptr(src.ptr)) self.mem_copy(T, src, dst.raw) else self.mem_transfer(T, src, dst.raw, .HtoD);
    return dst;
}
pub fn mem_alloc(self: *Self, T: type, n: usize) ![]T {
    if (n == 0) return &.{};
    if (T == usize) return self.host_alloc(T, n); // NDArray.gather fills its offsets with a host loop
    var ptr: ?*anyopaque = null;
    if (c.zg_hip_alloc(self.ctx, n * @sizeOf(T), &ptr) != 0) return Error.DeviceOOM;
    const p: [*]T = @ptrCast(@alignCast(ptr.?));
    return p[0..n];
}
pub fn mem_alloc_byte_mask(self: *Self, n: usize) ![]u8 {
    return self.mem_alloc(u8, @divFloor(n - 1, 8) + 1);
}
pub fn mem_free(self: *Self, slice: anytype) void {
    if (slice.len == 0) return;
    if (std.meta.Elem(@TypeOf(slice)) == usize) return check(c.zg_hip_host_free(self.ctx, @constCast(@ptrCast(slice.ptr))));
    check(c.zg_hip_free(self.ctx, @constCast(@ptrCast(slice.ptr))));
}
pub fn mem_dupe(self: *Self, T: type, src: []const T) ![]T {
    const dst = try self.mem_alloc(T, src.len);
    self.mem_copy(T, src, dst);
    return dst;
}
pub fn mem_scratch(self: *Self, T: type, n: usize) []T {
    if (n == 0) return &.{};
    var ptr: ?*anyopaque = null;
    check(c.zg_hip_mem_scratch(self.ctx, n * @sizeOf(T), &ptr)); // grow-only, src/allocators/caching_allocator.zig:133-156
    const p: [*]T = @ptrCast(@alignCast(ptr.?));
    return p[0..n];
}
pub fn mem_fill(self: *const Self, T: type, slice: []T, value: T) void {
    switch (T) {
        f32 => check(c.zg_hip_mem_fill(self.ctx, slice.ptr, slice.len, value)),
        u8 => check(c.zg_hip_mem_fill_u8(self.ctx, slice.ptr, slice.len, value)),
        usize => check(c.zg_hip_mem_fill_u64(self.ctx, @ptrCast(slice.ptr), slice.len, value)),
        else => @compileError("HipDevice.mem_fill: unsupported element type " ++ @typeName(T)),
    }
    if (T == usize) self.sync(); // host-visible memory: a host loop may read it next
}
pub fn mem_copy(self: *const Self, T: type, src: []const T, dst: []T) void {
    check(c.zg_hip_memcpy_d2d(self.ctx, dst.ptr, src.ptr, src.len * @sizeOf(T)));
    if (T == usize) self.sync(); // host-visible memory: a host loop may read it next
}
pub fn mem_transfer(self: *const Self, T: type, src: []const T, dst: []T, dir: TransferDirection) void {
    const n = src.len * @sizeOf(T);
    switch (dir) {
        .HtoD => check(c.zg_hip_memcpy_h2d(self.ctx, dst.ptr, src.ptr, n)),
        .DtoH => check(c.zg_hip_memcpy_d2h(self.ctx, dst.ptr, src.ptr, n)), // blocks: NDTensor.get reads right after
        .DtoD => check(c.zg_hip_memcpy_d2d(self.ctx, dst.ptr, src.ptr, n)),
    }
    if (T == usize and dir == .DtoD) self.sync(); // the other two directions have waited already
}
pub fn mem_sequence(self: *const Self, T: type, slice: []T, initial: T, step: T) void {
    comptime std.debug.assert(T == f32);
    check(c.zg_hip_mem_sequence(self.ctx, slice.ptr, slice.len, initial, step));
}
pub fn mem_random(self: *const Self, T: type, slice: []T, op: RandType, rand: std.Random) void {
    // Generate on the host with the caller's generator, exactly as HostDevice does
    // (src/device/host_device.zig:931-945), then copy up: bit-identical initial weights on both devices.
    comptime std.debug.assert(T == f32);
    const tmp = std.heap.page_allocator.alloc(T, slice.len) catch @panic("mem_random: host OOM");
    defer std.heap.page_allocator.free(tmp);
    switch (op) {
        .uniform => for (tmp) |*e| {
            e.* = rand.float(T);
        },
        .normal => for (tmp) |*e| {
            e.* = rand.floatNorm(T);
        },
        .kaiming => |fan| {
            const std_dev = @sqrt(2.0 / @as(T, @floatFromInt(fan)));
            for (tmp) |*e| e.* = rand.floatNorm(T) * std_dev;
        },
    }
    self.mem_transfer(T, tmp, slice, .HtoD);
}
pub fn mem_take(self: *const Self, T: type, src: []const T, idxs: []const usize, dst: []T) void {
    comptime std.debug.assert(T == f32);
    check(c.zg_hip_mem_take(self.ctx, src.ptr, src.len, @ptrCast(idxs.ptr), idxs.len, dst.ptr));
}

// --------------------------------------------------------------------------------------------------
// ops: one method per opspec name.  f32 only; any other T is a compile error at the call site.
// --------------------------------------------------------------------------------------------------
fn only_f32(T: type) void {
    if (T != f32) @compileError("HipDevice implements f32 ops; got " ++ @typeName(T));
}

/// z = x o y with the reference's broadcasting (src/device/host_device.zig:975-1019).  An operand of one element
/// that is not device memory is a scalar on the caller's stack (NDArray.add_scalar: `.y = &.{s}`,
/// src/ndarray.zig:247-257) and is passed by value.
const BinaryOp = enum { add, sub, mul, div };
fn binary(self: *const Self, comptime op: BinaryOp, x: []const f32, y: []const f32, z: []f32) void {
    const x_host = x.len == 1 and !self.is_device_ptr(x.ptr);
    const y_host = y.len == 1 and !self.is_device_ptr(y.ptr);
    if (x_host and y_host) {
        // both operands on the host: the one result is formed where HostDevice forms it, the same fp32 operation
        const v: f32 = switch (op) {
            .add => x[0] + y[0],
            .sub => x[0] - y[0],
            .mul => x[0] * y[0],
            .div => x[0] / y[0],
        };
        return check(c.zg_hip_mem_fill(self.ctx, z.ptr, z.len, v));
    }
    if (x_host or y_host) {
        const vec = if (y_host) x else y;
        const s = if (y_host) y[0] else x[0];
        const lhs: c_int = @intFromBool(x_host);
        return check(switch (op) {
            .add => c.zg_hip_add_scalar(self.ctx, vec.ptr, vec.len, s, lhs, z.ptr),
            .sub => c.zg_hip_sub_scalar(self.ctx, vec.ptr, vec.len, s, lhs, z.ptr),
            .mul => c.zg_hip_mul_scalar(self.ctx, vec.ptr, vec.len, s, lhs, z.ptr),
            .div => c.zg_hip_div_scalar(self.ctx, vec.ptr, vec.len, s, lhs, z.ptr),
        });
    }
    check(switch (op) {
        .add => c.zg_hip_add(self.ctx, x.ptr, x.len, y.ptr, y.len, z.ptr, z.len),
        .sub => c.zg_hip_sub(self.ctx, x.ptr, x.len, y.ptr, y.len, z.ptr, z.len),
        .mul => c.zg_hip_mul(self.ctx, x.ptr, x.len, y.ptr, y.len, z.ptr, z.len),
        .div => c.zg_hip_div(self.ctx, x.ptr, x.len, y.ptr, y.len, z.ptr, z.len),
    });
}
pub fn add(self: *const Self, T: type, p: opspec.add(T)) void {
    comptime only_f32(T);
    self.binary(.add, p.x, p.y, p.z);
}
pub fn sub(self: *const Self, T: type, p: opspec.sub(T)) void {
    comptime only_f32(T);
    self.binary(.sub, p.x, p.y, p.z);
}
pub fn mul(self: *const Self, T: type, p: opspec.mul(T)) void {
    comptime only_f32(T);
    self.binary(.mul, p.x, p.y, p.z);
}
pub fn div(self: *const Self, T: type, p: opspec.div(T)) void {
    comptime only_f32(T);
    self.binary(.div, p.x, p.y, p.z);
}
pub fn dot(self: *const Self, T: type, p: opspec.dot(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_dot(self.ctx, p.x.ptr, p.y.ptr, p.x.len, p.z.ptr));
}
pub fn matvec(self: *const Self, T: type, p: opspec.matvec(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_matvec(self.ctx, p.A.ptr, p.x.ptr, p.y.ptr, p.m, p.n, @intFromBool(p.trans_a), p.alpha, p.beta));
}
pub fn matmul(self: *const Self, T: type, p: opspec.matmul(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_matmul(self.ctx, p.A.ptr, p.B.ptr, p.C.ptr, p.m, p.n, p.k, @intFromBool(p.trans_a), @intFromBool(p.trans_b), p.lda, p.ldb, p.ldc, p.alpha, p.beta));
}
pub fn bmm_acc(self: *const Self, T: type, p: opspec.bmm_acc(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_bmm_acc(self.ctx, p.A.ptr, @ptrCast(p.A_shape.ptr), p.B.ptr, @ptrCast(p.B_shape.ptr), p.C.ptr, @ptrCast(p.C_shape.ptr), @intFromBool(p.trans_a), @intFromBool(p.trans_b), p.lda, p.ldb, p.ldc, p.alpha, p.beta));
}
pub fn outer(self: *const Self, T: type, p: opspec.outer(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_outer(self.ctx, p.x.ptr, p.x.len, p.y.ptr, p.y.len, p.A.ptr, p.alpha));
}
pub fn transpose(self: *const Self, T: type, p: opspec.transpose(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_transpose(self.ctx, p.A.ptr, p.B.ptr, p.m, p.n, p.alpha));
}
pub fn axpy(self: *const Self, T: type, p: opspec.axpy(T)) void {
    comptime only_f32(T);
    const on_device = self.is_device_ptr(p.alpha);
    check(c.zg_hip_axpy(self.ctx, p.x.ptr, p.y.ptr, p.x.len, p.alpha, @intFromBool(on_device)));
}
pub fn sum(self: *const Self, T: type, p: opspec.sum(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_sum(self.ctx, p.x.ptr, p.x.len, p.y.ptr));
}
pub fn scale(self: *const Self, T: type, p: opspec.scale(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_scale(self.ctx, p.x.ptr, p.x.len, p.alpha));
}
pub fn nrm2(self: *const Self, T: type, p: opspec.nrm2(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_nrm2(self.ctx, p.x.ptr, p.x.len, p.y.ptr));
}
pub fn clip_nrm2(self: *const Self, T: type, p: opspec.clip_nrm2(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_clip_nrm2(self.ctx, p.x.ptr, p.x.len, p.max_norm, p.delta));
}
pub fn pow_fwd(self: *const Self, T: type, p: opspec.pow_fwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_pow_fwd(self.ctx, p.x.ptr, p.y.ptr, p.x.len, p.exp));
}
pub fn pow_fwd_(self: *const Self, T: type, p: opspec.pow_fwd_(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_pow_fwd(self.ctx, p.x.ptr, p.x.ptr, p.x.len, p.exp));
}
pub fn pow_bwd(self: *const Self, T: type, p: opspec.pow_bwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_pow_bwd(self.ctx, p.x.ptr, p.x_g.ptr, p.y_g.ptr, p.x.len, p.exp, p.eps));
}
pub fn sqrt_fwd(self: *const Self, T: type, p: opspec.sqrt_fwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_sqrt_fwd(self.ctx, p.x.ptr, p.y.ptr, p.x.len));
}
pub fn sqrt_fwd_(self: *const Self, T: type, p: opspec.sqrt_fwd_(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_sqrt_fwd(self.ctx, p.x.ptr, p.x.ptr, p.x.len));
}
pub fn sqrt_bwd(self: *const Self, T: type, p: opspec.sqrt_bwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_sqrt_bwd(self.ctx, p.x.ptr, p.x_g.ptr, p.y_g.ptr, p.x.len, p.eps));
}
pub fn rsqrt_fwd(self: *const Self, T: type, p: opspec.rsqrt_fwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_rsqrt_fwd(self.ctx, p.x.ptr, p.y.ptr, p.x.len, p.eps));
}
pub fn rsqrt_bwd(self: *const Self, T: type, p: opspec.rsqrt_bwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_rsqrt_bwd(self.ctx, p.x.ptr, p.x_g.ptr, p.y_g.ptr, p.x.len, p.eps));
}
pub fn exp_fwd(self: *const Self, T: type, p: opspec.exp_fwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_exp_fwd(self.ctx, p.x.ptr, p.y.ptr, p.x.len));
}
pub fn exp_bwd(self: *const Self, T: type, p: opspec.exp_bwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_exp_bwd(self.ctx, p.x_g.ptr, p.y.ptr, p.y_g.ptr, p.x_g.len));
}
pub fn relu_fwd(self: *const Self, T: type, p: opspec.relu_fwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_relu_fwd(self.ctx, p.x.ptr, p.y.ptr, p.x.len));
}
pub fn relu_bwd(self: *const Self, T: type, p: opspec.relu_bwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_relu_bwd(self.ctx, p.x.ptr, p.x_g.ptr, p.y_g.ptr, p.x.len));
}
pub fn relu_inplace_bwd(self: *const Self, T: type, p: opspec.relu_inplace_bwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_relu_inplace_bwd(self.ctx, p.x.ptr, p.x_g.ptr, p.x.len));
}
pub fn tanh_fwd(self: *const Self, T: type, p: opspec.tanh_fwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_tanh_fwd(self.ctx, p.x.ptr, p.y.ptr, p.x.len));
}
pub fn tanh_bwd(self: *const Self, T: type, p: opspec.tanh_bwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_tanh_bwd(self.ctx, p.x_g.ptr, p.y.ptr, p.y_g.ptr, p.x_g.len));
}
pub fn tanh_inplace_bwd(self: *const Self, T: type, p: opspec.tanh_inplace_bwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_tanh_inplace_bwd(self.ctx, p.x.ptr, p.x_g.ptr, p.x.len));
}
pub fn sigm_fwd(self: *const Self, T: type, p: opspec.sigm_fwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_sigm_fwd(self.ctx, p.x.ptr, p.y.ptr, p.x.len));
}
pub fn sigm_bwd(self: *const Self, T: type, p: opspec.sigm_bwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_sigm_bwd(self.ctx, p.x_g.ptr, p.y.ptr, p.y_g.ptr, p.x_g.len));
}
pub fn sigm_inplace_bwd(self: *const Self, T: type, p: opspec.sigm_inplace_bwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_sigm_inplace_bwd(self.ctx, p.x.ptr, p.x_g.ptr, p.x.len));
}
pub fn max_fwd(self: *const Self, T: type, p: opspec.max_fwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_max_fwd(self.ctx, p.x.ptr, p.x.len, p.y.ptr));
}
pub fn max_bwd(self: *const Self, T: type, p: opspec.max_bwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_max_bwd(self.ctx, p.x.ptr, p.x_g.ptr, p.x.len, p.y.ptr, p.y_g.ptr));
}
pub fn clamp_fwd(self: *const Self, T: type, p: opspec.clamp_fwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_clamp_fwd(self.ctx, p.x.ptr, p.y.ptr, p.x.len, p.min, p.max));
}
pub fn clamp_bwd(self: *const Self, T: type, p: opspec.clamp_bwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_clamp_bwd(self.ctx, p.x.ptr, p.x_g.ptr, p.y_g.ptr, p.x.len, p.min, p.max));
}
pub fn unbroadcast(self: *Self, T: type, p: opspec.unbroadcast(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_unbroadcast(self.ctx, p.x.ptr, @ptrCast(p.x_shape.ptr), p.x_shape.len, p.y.ptr, @ptrCast(p.y_shape.ptr), p.y_shape.len, p.scratch.ptr, p.scratch.len, p.alpha, p.beta));
}
pub fn broadcast(self: *const Self, T: type, p: opspec.broadcast(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_broadcast(self.ctx, p.x.ptr, p.x.len, p.y.ptr, p.y.len, p.alpha, p.beta));
}
pub fn sum_along(self: *const Self, T: type, p: opspec.sum_along(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_sum_along(self.ctx, p.x.ptr, @ptrCast(p.x_shape.ptr), p.x_shape.len, p.y.ptr, p.y.len, p.dim, p.alpha, p.beta));
}
pub fn max_along(self: *const Self, T: type, p: opspec.max_along(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_max_along(self.ctx, p.x.ptr, @ptrCast(p.x_shape.ptr), p.x_shape.len, p.y.ptr, p.y.len, p.dim));
}
pub fn scatter_add(self: *const Self, T: type, p: opspec.scatter_add(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_scatter_add(self.ctx, p.src.ptr, @ptrCast(p.offsets.ptr), p.src.len, p.dst.ptr, p.dst.len));
}
pub fn scatter_add_csr(self: *const Self, T: type, p: opspec.scatter_add_csr(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_scatter_add_csr(self.ctx, p.src.ptr, @ptrCast(p.row_ptr.ptr), p.src.len, p.dst.ptr, p.dst.len));
}
pub fn segment_sum_csr(self: *const Self, T: type, p: opspec.segment_sum_csr(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_segment_sum_csr(self.ctx, p.src.ptr, p.src.len, @ptrCast(p.row_offsets.ptr), p.dst.len, p.dst.ptr));
}
pub fn scatter_gcn_deg_scaled(self: *const Self, T: type, p: opspec.scatter_gcn_deg_scaled(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_scatter_gcn_deg_scaled(self.ctx, p.dst.ptr, p.h.ptr, p.deg.ptr, @ptrCast(p.src_indices.ptr), @ptrCast(p.tgt_indices.ptr), p.stride, p.n_edge, p.deg.len));
}
pub fn scatter_gcn_deg_scaled_bwd(self: *const Self, T: type, p: opspec.scatter_gcn_deg_scaled_bwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_scatter_gcn_deg_scaled_bwd(self.ctx, p.grad_output.ptr, p.h.ptr, p.deg.ptr, @ptrCast(p.src_indices.ptr), @ptrCast(p.tgt_indices.ptr), p.grad_h.ptr, p.grad_deg.ptr, p.stride, p.n_edge, p.deg.len));
}

// New op names for what the reference computes with host loops over `.raw`.  Their parameter structs are in
// zig/opspec_additions.zig (to be appended to src/device/opspec.zig); the call sites that switch to dispatch:
//   smce_fwd / smce_bwd / smce_label_fwd / smce_label_bwd   src/nn/loss.zig:130-215
//   softmax_fwd / softmax_bwd                                src/nn/loss.zig:217-257
//   smooth_l1_fwd / smooth_l1_bwd / mse_fwd / mse_bwd        src/nn/loss.zig:94-127, 259-305
//   sgd_step / adam_step                                     src/nn/optim.zig:100-122, 177-234
//   argmax_along, gather_offsets, index_select_fwd / _bwd    examples/mnist/src/main-simple.zig:124, src/ndarray.zig:607-624,
//                                                            src/ndtensor.zig:1437-1513
pub fn argmax_along(self: *const Self, T: type, p: opspec.argmax_along(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_argmax_along(self.ctx, p.x.ptr, @ptrCast(p.x_shape.ptr), p.x_shape.len, @ptrCast(p.y.ptr), p.y.len, p.dim));
    self.sync(); // `y` is host-visible index memory: the caller's loop reads it next
}
/// The offsets loop of NDArray.gather (src/ndarray.zig:607-624) on the device.  `p.check` reads the status back.
pub fn gather_offsets(self: *const Self, T: type, p: opspec.gather_offsets(T)) !void {
    comptime only_f32(T);
    var status: c_int = 0;
    const status_ptr: ?*c_int = if (p.check) &status else null;
    const rc = c.zg_hip_gather_offsets(self.ctx, @ptrCast(p.src_shape.ptr), @ptrCast(p.idx_shape.ptr), p.src_shape.len, @ptrCast(p.indices.ptr), p.dim, @ptrCast(p.offsets.ptr), status_ptr);
    if (status == 1) return error.InvalidIndexShape;
    if (status == 2) return error.IndexOutOfBounds;
    check(rc);
}
pub fn index_select_fwd(self: *const Self, T: type, p: opspec.index_select_fwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_index_select_fwd(self.ctx, p.src.ptr, p.src.len, @ptrCast(p.indices.ptr), p.indices.len, p.stride, p.dst.ptr));
}
pub fn index_select_bwd(self: *const Self, T: type, p: opspec.index_select_bwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_index_select_bwd(self.ctx, p.y_grad.ptr, @ptrCast(p.indices.ptr), p.indices.len, p.stride, p.x_grad.ptr, p.x_grad.len));
}
pub fn smce_label_fwd(self: *const Self, T: type, p: opspec.smce_label_fwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_smce_label_fwd(self.ctx, p.logits.ptr, @ptrCast(p.labels.ptr), p.lse.ptr, p.loss.ptr, p.rows, p.cols));
}
pub fn smce_label_bwd(self: *const Self, T: type, p: opspec.smce_label_bwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_smce_label_bwd(self.ctx, p.logits.ptr, @ptrCast(p.labels.ptr), p.lse.ptr, p.grad.ptr, p.rows, p.cols, @intFromBool(p.accumulate)));
}
pub fn softmax_fwd(self: *const Self, T: type, p: opspec.softmax_fwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_softmax_fwd(self.ctx, p.x.ptr, p.y.ptr, p.rows, p.cols));
}
pub fn softmax_bwd(self: *const Self, T: type, p: opspec.softmax_bwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_softmax_bwd(self.ctx, p.y.ptr, p.y_g.ptr, p.x_g.ptr, p.rows, p.cols));
}
/// NDArray.gather (src/ndarray.zig:593-633) as one device op: the offsets (kept for the backward's scatter_add) and
/// the gathered values.  `p.check` reads the out-of-bounds status back (one blocking 4-byte copy).
pub fn gather(self: *const Self, T: type, p: opspec.gather(T)) !void {
    comptime only_f32(T);
    var status: c_int = 0;
    const status_ptr: ?*c_int = if (p.check) &status else null;
    const rc = c.zg_hip_gather(self.ctx, p.src.ptr, @ptrCast(p.src_shape.ptr), @ptrCast(p.idx_shape.ptr), p.src_shape.len, @ptrCast(p.indices.ptr), p.dim, @ptrCast(p.offsets.ptr), p.dst.ptr, status_ptr);
    if (status == 1) return error.InvalidIndexShape;
    if (status == 2) return error.IndexOutOfBounds;
    check(rc);
}
pub fn smce_fwd(self: *const Self, T: type, p: opspec.smce_fwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_smce_fwd(self.ctx, p.logits.ptr, p.target.ptr, p.probs.ptr, p.loss.ptr, p.rows, p.cols));
}
pub fn smce_bwd(self: *const Self, T: type, p: opspec.smce_bwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_smce_bwd(self.ctx, p.probs.ptr, p.target.ptr, p.grad.ptr, p.rows, p.cols));
}
/// smce_fwd and the backward of the scalar loss in one call (upstream gradient 1): p.grad (+)= (probs - target)/rows.
pub fn smce_fwd_bwd(self: *const Self, T: type, p: opspec.smce_fwd_bwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_smce_fwd_bwd(self.ctx, p.logits.ptr, p.target.ptr, p.probs.ptr, p.loss.ptr, p.grad.ptr, p.rows, p.cols, @intFromBool(p.accumulate)));
}
pub fn smooth_l1_fwd(self: *const Self, T: type, p: opspec.smooth_l1_fwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_smooth_l1_fwd(self.ctx, p.pred.ptr, p.target.ptr, p.pred.len, p.beta, p.loss.ptr));
}
/// smooth_l1_fwd and the backward of the scalar loss in one call: p.grad (+)= d loss / d pred.
pub fn smooth_l1_fwd_bwd(self: *const Self, T: type, p: opspec.smooth_l1_fwd_bwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_smooth_l1_fwd_bwd(self.ctx, p.pred.ptr, p.target.ptr, p.grad.ptr, p.pred.len, p.beta, p.loss.ptr, @intFromBool(p.accumulate)));
}
pub fn smooth_l1_bwd(self: *const Self, T: type, p: opspec.smooth_l1_bwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_smooth_l1_bwd(self.ctx, p.pred.ptr, p.target.ptr, p.grad.ptr, p.pred.len, p.beta));
}
pub fn mse_fwd(self: *const Self, T: type, p: opspec.mse_fwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_mse_fwd(self.ctx, p.pred.ptr, p.target.ptr, p.pred.len, p.loss.ptr));
}
pub fn mse_bwd(self: *const Self, T: type, p: opspec.mse_bwd(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_mse_bwd(self.ctx, p.pred.ptr, p.target.ptr, p.grad.ptr, p.pred.len));
}
pub fn sgd_step(self: *const Self, T: type, p: opspec.sgd_step(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_sgd_step(self.ctx, p.param.ptr, p.grad.ptr, p.param.len, p.lr, @intFromBool(p.clip), p.max_norm, p.delta));
}
pub fn adam_step(self: *const Self, T: type, p: opspec.adam_step(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_adam_step(self.ctx, p.param.ptr, p.grad.ptr, p.m.ptr, p.v.ptr, p.param.len, @intCast(p.t), p.lr, p.beta1, p.beta2, p.epsilon, @intFromBool(p.clip), p.max_norm, p.delta));
}

/// Optimizer.step() over a whole parameter list (src/nn/optim.zig:100-122, :177-234), optionally followed by
/// model.zero_grad(): small tensors share launches.  `p.params`, `p.grads` (and `p.ms`, `p.vs`) are slices of
/// device pointers, `p.lens` their element counts; Adam's `p.lr_t` holds one step size per tensor
/// (`adam_lr_t` with that tensor's counter), in host memory unless `p.lr_t_in_memory`.
pub fn sgd_step_multi(self: *const Self, T: type, p: opspec.sgd_step_multi(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_sgd_step_multi(self.ctx, p.params.len, p.params.ptr, p.grads.ptr, p.lens.ptr, p.lr, @intFromBool(p.clip), p.max_norm, p.delta, @intFromBool(p.zero_grads)));
}
pub fn adam_step_multi(self: *const Self, T: type, p: opspec.adam_step_multi(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_adam_step_multi(self.ctx, p.params.len, p.params.ptr, p.grads.ptr, p.ms.ptr, p.vs.ptr, p.lens.ptr, p.lr_t.ptr, @intFromBool(p.lr_t_in_memory), p.beta1, p.beta2, p.epsilon, @intFromBool(p.clip), p.max_norm, p.delta, @intFromBool(p.zero_grads)));
}

/// Both destination orderings of an edge list that does not change between calls (the dataset's graph), built
/// once; `scatter_add_planned`, `scatter_gcn_deg_scaled_planned` and `scatter_gcn_deg_scaled_bwd_planned` then
/// return what the ops that take bare index slices return, without sorting the edges again on every call.
pub const EdgePlan = struct {
    ctx: *c.zg_hip_ctx,
    plan: ?*c.zg_hip_edge_plan = null,

    pub fn init(device: *const Self, src_indices: []const usize, tgt_indices: []const usize, n_nodes: usize) EdgePlan {
        var self = EdgePlan{ .ctx = device.ctx };
        check(c.zg_hip_edge_plan_create(device.ctx, @ptrCast(src_indices.ptr), @ptrCast(tgt_indices.ptr), src_indices.len, n_nodes, &self.plan));
        return self;
    }
    pub fn deinit(self: *EdgePlan) void {
        check(c.zg_hip_edge_plan_free(self.ctx, self.plan));
        self.plan = null;
    }
};
pub fn scatter_add_planned(self: *const Self, T: type, p: opspec.scatter_add_planned(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_scatter_add_planned(self.ctx, p.src.ptr, p.plan.plan, p.dst.ptr, @intFromBool(p.accumulate)));
}
pub fn scatter_gcn_deg_scaled_planned(self: *const Self, T: type, p: opspec.scatter_gcn_deg_scaled_planned(T)) void {
    comptime only_f32(T);
    const bias: ?[*]const T = if (p.bias) |b| b.ptr else null;  // the layer's tail: + bias, then relu when asked
    check(c.zg_hip_scatter_gcn_deg_scaled_planned(self.ctx, p.dst.ptr, p.h.ptr, p.deg.ptr, p.plan.plan, bias, @intFromBool(p.relu), p.stride, @intFromBool(p.accumulate)));
}
pub fn scatter_gcn_deg_scaled_bwd_planned(self: *const Self, T: type, p: opspec.scatter_gcn_deg_scaled_bwd_planned(T)) void {
    comptime only_f32(T);
    const gd: ?[*]T = if (p.grad_deg) |g| g.ptr else null; // optional: the degrees are data of the graph
    check(c.zg_hip_scatter_gcn_deg_scaled_bwd_planned(self.ctx, p.grad_output.ptr, p.h.ptr, p.deg.ptr, p.plan.plan, p.grad_h.ptr, gd, p.stride, @intFromBool(p.accumulate)));
}

/// A Linear layer's forward in one launch: y = act(x . w^T + bias), the arithmetic of `bmm_acc(trans_b)` +
/// `bias.add_` + `relu_` (examples/mnist/src/model.zig:104-110, :38-46).  `p.bias` is an optional slice.
pub fn linear_fwd(self: *const Self, T: type, p: opspec.linear_fwd(T)) void {
    comptime only_f32(T);
    const bias: ?[*]const T = if (p.bias) |b| b.ptr else null;
    check(c.zg_hip_linear_fwd(self.ctx, p.x.ptr, p.w.ptr, bias, p.y.ptr, p.batch, p.fan_in, p.fan_out, @intFromBool(p.relu)));
}
/// The input gradient of a Linear layer with the ReLU backward of the layer before it in one launch:
/// gx = (accumulate ? gx : 0) + gy . w, zeroed where `p.act_in` (that ReLU's output, optional) is <= 0:
/// the dA product of BmmAccBwd (src/ndtensor.zig:1092-1136) + relu_inplace_bwd (src/device/host_device.zig:543-547).
pub fn linear_bwd_input(self: *const Self, T: type, p: opspec.linear_bwd_input(T)) void {
    comptime only_f32(T);
    const act: ?[*]const T = if (p.act_in) |a| a.ptr else null;
    check(c.zg_hip_linear_bwd_input(self.ctx, p.gy.ptr, p.w.ptr, act, p.gx.ptr, p.batch, p.fan_in, p.fan_out, @intFromBool(p.accumulate)));
}
/// The whole backward of a Linear layer for a final output gradient: gw += gy^T . x, gb += column sums of gy
/// (`p.gb` optional), gx = gy . w zeroed where `p.act_in` <= 0 (`p.gx`, `p.act_in` optional): the two products of
/// BmmAccBwd (src/ndtensor.zig:1092-1136), the bias's unbroadcast and relu_inplace_bwd of the layer before.
pub fn linear_bwd(self: *const Self, T: type, p: opspec.linear_bwd(T)) void {
    comptime only_f32(T);
    const act: ?[*]const T = if (p.act_in) |a| a.ptr else null;
    const gb: ?[*]T = if (p.gb) |b| b.ptr else null;
    const gx: ?[*]T = if (p.gx) |g| g.ptr else null;
    check(c.zg_hip_linear_bwd(self.ctx, p.gy.ptr, p.x.ptr, p.w.ptr, act, p.gw.ptr, gb, gx, p.batch, p.fan_in, p.fan_out));
}

/// Adam update whose `lr_t` is read from memory when the kernel runs (`p.lr_t` points to device memory or
/// to `mem_alloc_indices`-style pinned host memory).  A step recorded with `capture.open()` can then be
/// replayed for every later step: the host only rewrites `lr_t` between replays.
pub fn adam_step_at(self: *const Self, T: type, p: opspec.adam_step_at(T)) void {
    comptime only_f32(T);
    check(c.zg_hip_adam_step_at(self.ctx, p.param.ptr, p.grad.ptr, p.m.ptr, p.v.ptr, p.param.len, p.lr_t.ptr, p.beta1, p.beta2, p.epsilon, @intFromBool(p.clip), p.max_norm, p.delta));
}

/// The ExecutionGraph of the reference's second device (src/device/cuda_device.zig:558-611), same four calls.
/// Between `open` and `save` every op is recorded instead of executed.  Cache blocks handed out or returned while
/// recording may be reused by later allocations of the same recording; whatever part of them is free at `save`
/// stays with the graph, so the recorded addresses remain private to it until `free`.
pub const ExecutionGraph = struct {
    ctx: *c.zg_hip_ctx,
    graph: ?*c.zg_hip_graph = null,
    open_now: bool = false,

    pub const RunError = error{ CaptureInProgress, UndefinedCapture };

    pub fn run(self: *ExecutionGraph) RunError!void {
        if (self.open_now) return error.CaptureInProgress;
        const g = self.graph orelse return error.UndefinedCapture;
        check(c.zg_hip_graph_run(self.ctx, g));
    }
    pub fn open(self: *ExecutionGraph, config: struct {}) void {
        _ = config;
        self.free();
        check(c.zg_hip_graph_open(self.ctx));
        self.open_now = true;
    }
    pub fn save(self: *ExecutionGraph) void {
        if (!self.open_now) return;
        var g: ?*c.zg_hip_graph = null;
        check(c.zg_hip_graph_save(self.ctx, &g));
        self.graph = g;
        self.open_now = false;
    }
    pub fn free(self: *ExecutionGraph) void {
        self.save();
        if (self.graph) |g| check(c.zg_hip_graph_free(self.ctx, g));
        self.graph = null;
    }
    pub fn empty(self: ExecutionGraph) bool {
        return self.graph == null;
    }
};

pub fn execution_graph(self: *const Self) ExecutionGraph {
    return .{ .ctx = self.ctx };
}

// Input staging (no counterpart in the reference, which uploads each batch with a blocking mem_transfer):
// upload the next batch from `mem_alloc_indices`-style pinned host memory on the copy stream while the current
// batch computes.  Order per step: compute_after_staging(), staging_after_compute(), staged_h2d(next batch),
// then the ops of the current step.
pub fn staged_h2d(self: *const Self, T: type, src_pinned: []const T, dst: []T) void {
    check(c.zg_hip_staged_h2d(self.ctx, dst.ptr, src_pinned.ptr, src_pinned.len * @sizeOf(T)));
}
pub fn staging_after_compute(self: *const Self) void {
    check(c.zg_hip_staging_after_compute(self.ctx));
}
pub fn compute_after_staging(self: *const Self) void {
    check(c.zg_hip_compute_after_staging(self.ctx));
}
pub fn staging_wait(self: *const Self) void {
    check(c.zg_hip_staging_wait(self.ctx));
}
