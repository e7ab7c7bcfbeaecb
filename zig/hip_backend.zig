//! aion backend shim over libaion_hip.so (include/aion_hip.h).
//!
//! NOT COMPILED in this repository: the build image has no Zig toolchain (aion pins
//! 0.18.0-dev.1180, build.zig.zon:28). It is the reference-side binding a maintainer adds under
//! src/aion/backend/hip/: it adapts the three seams a device backend plugs into -
//! `Backend.VTable` + `Session.VTable` (backend/backend.zig:24-107), `DeviceMemory.VTable`
//! (runtime/device_memory.zig:36-108) and the `quant_block_order` constant
//! (api/gpu_device.zig:24-25) - onto the C ABI, mirroring backend/gpu/backend.zig:459-548.
//! Host code stays Zig; HIP is reached only through the @cImport below.
const std = @import("std");
const c = @cImport(@cInclude("aion_hip.h"));

const backend_mod = @import("../backend.zig");
const types = @import("../types.zig");
const executable = @import("../../runtime/executable.zig");
const dm = @import("../../runtime/device_memory.zig");
const device_store = @import("../../runtime/device_store.zig");
const tensor_store = @import("../../runtime/tensor_store.zig");

const BackendError = types.BackendError;
const ExecuteProgramError = backend_mod.ExecuteProgramError;

fn check(rc: c_int) ExecuteProgramError!void {
    return switch (rc) {
        c.AIONHIP_OK => {},
        c.AIONHIP_INVALID_ARGUMENT => BackendError.InvalidArgument,
        c.AIONHIP_UNSUPPORTED => BackendError.Unsupported,
        c.AIONHIP_OUT_OF_MEMORY => tensor_store.StoreError.OutOfMemory,
        else => BackendError.ExecutionFailed,
    };
}

pub const HipBackend = struct {
    ctx: *c.aionhip_ctx,
    allocator: std.mem.Allocator,
    /// Re-laid weights, keyed by the device handle of the packed tensor (weights are immutable
    /// params, graph/graph.zig:55-58, so the key never goes stale while the tensor lives).
    weights: std.AutoHashMap(u64, *c.aionhip_weight),

    /// This backend keeps aion's packed blocks as they are and re-lays privately.
    pub const quant_block_order: types.QuantBlockOrder = .row_major;

    pub fn init(allocator: std.mem.Allocator, device_index: c_int) !HipBackend {
        var ctx: ?*c.aionhip_ctx = null;
        if (c.aionhip_create(device_index, null, &ctx) != c.AIONHIP_OK) return error.BackendUnavailable;
        return .{ .ctx = ctx.?, .allocator = allocator, .weights = std.AutoHashMap(u64, *c.aionhip_weight).init(allocator) };
    }

    pub fn deinit(self: *HipBackend) void {
        var it = self.weights.valueIterator();
        while (it.next()) |w| c.aionhip_weight_free(self.ctx, w.*);
        self.weights.deinit();
        c.aionhip_destroy(self.ctx);
    }

    // ---- DeviceMemory.VTable (discrete; maxBindingBytes = null -> tensors are never chunked)
    fn dmModel(_: *anyopaque) dm.MemoryModel {
        return .discrete;
    }
    fn dmAlloc(p: *anyopaque, bytes: usize, alignment: usize) dm.DeviceError!dm.DeviceHandle {
        const self: *HipBackend = @ptrCast(@alignCast(p));
        var h: u64 = 0;
        if (c.aionhip_alloc(self.ctx, bytes, alignment, &h) != c.AIONHIP_OK) return dm.DeviceError.OutOfMemory;
        return h;
    }
    fn dmFree(p: *anyopaque, h: dm.DeviceHandle) void {
        const self: *HipBackend = @ptrCast(@alignCast(p));
        if (self.weights.fetchRemove(h)) |kv| c.aionhip_weight_free(self.ctx, kv.value);
        c.aionhip_free(self.ctx, h);
    }
    fn dmH2D(p: *anyopaque, h: dm.DeviceHandle, off: usize, src: []const u8) dm.DeviceError!void {
        const self: *HipBackend = @ptrCast(@alignCast(p));
        if (c.aionhip_h2d(self.ctx, h, off, src.ptr, src.len) != c.AIONHIP_OK) return dm.DeviceError.CopyFailed;
    }
    fn dmD2H(p: *anyopaque, dst: []u8, h: dm.DeviceHandle, off: usize) dm.DeviceError!void {
        const self: *HipBackend = @ptrCast(@alignCast(p));
        if (c.aionhip_d2h(self.ctx, dst.ptr, h, off, dst.len) != c.AIONHIP_OK) return dm.DeviceError.CopyFailed;
    }
    fn dmD2D(p: *anyopaque, dst: dm.DeviceHandle, doff: usize, src: dm.DeviceHandle, soff: usize, bytes: usize) dm.DeviceError!void {
        const self: *HipBackend = @ptrCast(@alignCast(p));
        if (c.aionhip_d2d(self.ctx, dst, doff, src, soff, bytes) != c.AIONHIP_OK) return dm.DeviceError.CopyFailed;
    }
    pub const devmem_vtable: dm.DeviceMemory.VTable = .{
        .model = dmModel, .alloc = dmAlloc, .free = dmFree, .copyH2D = dmH2D, .copyD2H = dmD2H, .copyD2D = dmD2D,
    };
    pub fn deviceMemory(self: *HipBackend) dm.DeviceMemory {
        return .{ .ctx = self, .vtable = &devmem_vtable };
    }

    // ---- weights: re-lay at first use, straight from the packed blocks already on the device
    fn weightFor(self: *HipBackend, store: device_store.DeviceStore, id: tensor_store.TensorId, layout: c_int) ExecuteProgramError!*c.aionhip_weight {
        const meta = try store.meta(id);
        const chunk = try store.acquireConst(id);
        defer store.releaseConst(chunk.token);
        if (self.weights.get(chunk.handle)) |w| return w;
        const n = if (layout == c.AIONHIP_ROWS_NK) meta.shape[0] else meta.shape[1];
        const k = if (layout == c.AIONHIP_ROWS_NK) meta.shape[1] else meta.shape[0];
        var w: ?*c.aionhip_weight = null;
        try check(c.aionhip_weight_from_device(self.ctx, @intFromEnum(meta.dtype), layout, n, k, 0, chunk.handle + chunk.offset, &w));
        self.weights.put(chunk.handle, w.?) catch return tensor_store.StoreError.OutOfMemory;
        return w.?;
    }

    fn addr(store: device_store.DeviceStore, id: tensor_store.TensorId, comptime mutable: bool) ExecuteProgramError!u64 {
        const ch = if (mutable) try store.acquireMut(id) else try store.acquireConst(id);
        if (mutable) store.releaseMut(ch.token) else store.releaseConst(ch.token);
        return ch.handle + ch.offset;
    }

    /// One step of a validated program (the reduced twin of backend/gpu/backend.zig:459-548).
    pub fn dispatchStep(self: *HipBackend, store: device_store.DeviceStore, step: executable.Step) ExecuteProgramError!void {
        switch (step) {
            .MatMul => |s| {
                const am = try store.meta(s.a);
                const m = rowsOf(am);
                const w = try self.weightFor(store, s.b, c.AIONHIP_KMAJOR_KN);
                try check(c.aionhip_step_matmul(self.ctx, w, m, try addr(store, s.a, false), 0, try addr(store, s.c, true), 0, s.alpha, s.beta));
            },
            .MatMulNT => |s| {
                const am = try store.meta(s.a);
                const w = try self.weightFor(store, s.b, c.AIONHIP_ROWS_NK);
                try check(c.aionhip_step_matmul_nt(self.ctx, w, rowsOf(am), try addr(store, s.a, false), 0, try addr(store, s.c, true), 0, s.alpha, s.beta));
            },
            .Attention => |s| {
                const qm = try store.meta(s.q);
                const km = try store.meta(s.k);
                const vm = try store.meta(s.v);
                var p: c.aionhip_attention = std.mem.zeroes(c.aionhip_attention);
                p.out = try addr(store, s.out, true);
                p.q = try addr(store, s.q, false);
                p.k = try addr(store, s.k, false);
                p.v = try addr(store, s.v, false);
                p.query_positions = if (s.query_positions) |t| try addr(store, t, false) else 0;
                p.kv_lengths = if (s.kv_lengths) |t| try addr(store, t, false) else 0;
                p.batch = qm.shape[0]; p.l_q = qm.shape[1]; p.h_q = qm.shape[2]; p.d_k = qm.shape[3];
                p.t_kv = km.shape[1]; p.h_kv = km.shape[2]; p.d_v = vm.shape[3];
                p.q_dtype = @intFromEnum(qm.dtype); p.kv_dtype = @intFromEnum(km.dtype);
                p.scale = s.scale; p.attn_logits_soft_cap = s.attn_logits_soft_cap;
                p.window_left = s.window.left; p.window_right = s.window.right; p.window_chunk = s.window.chunk;
                // a rolling sequence cache reads key t from row t % capacity (cpu/exec/attention.zig:1537-1546)
                p.rolling = if (store.sequenceCachePolicyInfo(s.k).kind == .rolling) 1 else 0;
                try check(c.aionhip_step_attention(self.ctx, &p));
            },
            .RMSNorm => |s| {
                const om = try store.meta(s.out);
                const gm = try store.meta(s.gamma);
                const cols = elemCount(gm);
                try check(c.aionhip_step_rmsnorm(self.ctx, try addr(store, s.out, true), try addr(store, s.x, false), try addr(store, s.gamma, false),
                    try addr(store, s.beta, false), if (s.residual) |r| try addr(store, r, false) else 0, elemCount(om) / cols, cols, s.eps));
            },
            .RoPE1D => |s| {
                const m = try store.meta(s.out);
                try check(c.aionhip_step_rope(self.ctx, try addr(store, s.out, true), try addr(store, s.x, false), try addr(store, s.positions, false),
                    m.shape[0], m.shape[1], m.shape[2], m.shape[3], s.base_frequency, s.scale_factor, s.rope_proportion));
            },
            .ArgMax => |s| {
                const m = try store.meta(s.x);
                const n = m.shape[m.rank - 1];
                try check(c.aionhip_step_argmax(self.ctx, try addr(store, s.out, true), try addr(store, s.x, false), elemCount(m) / n, n));
            },
            // ElemwiseBinary(add | gate gelu), Gather(axis 0), Cast(f32->f16), SequenceAppend map to
            // aionhip_step_add / _gate_gelu / _gather_rows / _cast_f32_f16 / _append_f16 the same way;
            // Optional launch-saving pattern matches over consecutive steps of a decode program (same results as
            // the separate steps; fall back to them on AIONHIP_UNSUPPORTED):
            //   RMSNorm, MatMul x3 (q,k,v), RoPE1D x2, Cast f16 x2, SequenceAppend x2 -> aionhip_step_rmsnorm_qkv_rope_append
            //   RMSNorm x3 (per head, q,k,v), RoPE1D x2, Cast f16 x2, SequenceAppend x2 -> aionhip_step_headnorm_rope_append
            //   RMSNorm, MatMul x2 (gate, up), gate(gelu), MatMul (down)             -> aionhip_step_rmsnorm_geglu_matmul
            //   RMSNorm, MatMul(s)                                                   -> aionhip_step_rmsnorm_matmul
            //   gate(gelu), MatMul                                                   -> aionhip_step_gate_matmul
            // Transfer steps go through deviceMemory() exactly as in backend/gpu/backend.zig:416-457.
            else => return BackendError.Unsupported,
        }
    }

    fn rowsOf(m: tensor_store.TensorMeta) usize {
        var r: usize = 1;
        for (0..m.rank - 1) |d| r *= m.shape[d];
        return r;
    }
    fn elemCount(m: tensor_store.TensorMeta) usize {
        var r: usize = 1;
        for (0..m.rank) |d| r *= m.shape[d];
        return r;
    }

    /// Session.execute: every step in order, asynchronously; readback (Transfer) is the sync point.
    pub fn runProgram(self: *HipBackend, store: device_store.DeviceStore, prog: *const executable.ExecutableProgram) ExecuteProgramError!void {
        for (prog.steps) |step| try self.dispatchStep(store, step);
    }

    /// Session.retireResources: wait for the stream before storage evicts tensors.
    pub fn retire(self: *HipBackend) void {
        _ = c.aionhip_sync(self.ctx);
    }
};
