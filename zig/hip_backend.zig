//! aion backend shim over libaion_hip.so (include/aion_hip.h).
//!
//! NOT COMPILED in this repository: the build image has no Zig toolchain (aion pins
//! 0.18.0-dev.1180, build.zig.zon:28). It is the reference-side binding a maintainer adds under
//! src/aion/backend/hip/: it adapts the three seams a device backend plugs into -
//! `Backend.VTable` + `Session.VTable` (backend/backend.zig:24-107), `DeviceMemory.VTable`
//! (runtime/device_memory.zig:36-108) and the `quant_block_order` constant
//! (api/gpu_device.zig:24-25) - onto the C ABI, following the shape of backend/gpu/backend.zig:186-270
//! (session over a placed store) and :459-548 (step dispatch). One addition outside this file:
//! `BackendKind` (backend/types.zig:4-11) gains a member `hip`, appended, which the compiler uses as the
//! placement of programs built for this backend (api/context.zig:135-183 registers the backend under it).
//! Host code stays Zig; HIP is reached only through the @cImport below.
const std = @import("std");
const c = @cImport(@cInclude("aion_hip.h"));

const backend_mod = @import("../backend.zig");
const types = @import("../types.zig");
const executable = @import("../../runtime/executable.zig");
const dm = @import("../../runtime/device_memory.zig");
const tensor_store = @import("../../runtime/tensor_store.zig");

const Backend = backend_mod.Backend;
const Session = backend_mod.Session;
const BackendError = types.BackendError;
const ExecuteProgramError = backend_mod.ExecuteProgramError;
const TensorStore = tensor_store.TensorStore;
const TensorId = tensor_store.TensorId;

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

    /// This backend keeps aion's packed blocks as they are and re-lays privately.
    pub const quant_block_order: types.QuantBlockOrder = .row_major;

    pub fn init(allocator: std.mem.Allocator, device_index: c_int) !HipBackend {
        var ctx: ?*c.aionhip_ctx = null;
        if (c.aionhip_create(device_index, null, &ctx) != c.AIONHIP_OK) return error.BackendUnavailable;
        return .{ .ctx = ctx.?, .allocator = allocator };
    }

    /// The owner calls this; the vtable's `deinit` is a no-op like backend/gpu/backend.zig:675-678.
    /// Sessions are destroyed first (each frees the re-laid weights it holds through this context).
    pub fn deinit(self: *HipBackend) void {
        c.aionhip_destroy(self.ctx);
    }

    // ---- Backend.VTable (backend/backend.zig:58-73)
    fn kindImpl(_: *anyopaque) types.BackendKind {
        return .hip;
    }
    fn nameImpl(_: *anyopaque) []const u8 {
        return std.mem.span(c.aionhip_name());
    }
    fn capsImpl(_: *anyopaque) types.BackendCaps {
        return .{ .fp16 = true, .int8 = true, .quant_q4 = true, .quant_q8 = true };
    }
    fn deinitImpl(_: *anyopaque) void {}
    fn createSessionImpl(p: *anyopaque, store: TensorStore) tensor_store.StoreError!Session {
        const self: *HipBackend = @ptrCast(@alignCast(p));
        const s = try HipSession.create(self, store);
        return .{ .ctx = @ptrCast(s), .vtable = &HipSession.session_vtable };
    }
    const vtable = Backend.VTable{ .kind = kindImpl, .name = nameImpl, .caps = capsImpl, .deinit = deinitImpl, .createSession = createSessionImpl };
    pub fn backend(self: *HipBackend) Backend {
        return .{ .ctx = @ptrCast(self), .vtable = &vtable };
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

    /// A session bound to one placed tensor store (backend/gpu/backend.zig:206-270). Tensors the store placed on
    /// this device answer `deviceChunk` (runtime/tensor_store.zig:150-201) with one chunk: the whole buffer.
    /// Execution is the library's: every step becomes one `aionhip_step` record (its attributes plus, per TensorId,
    /// address, dtype and shape) and `aionhip_session_execute` dispatches, keeps the re-laid weights and folds the
    /// launch-saving step patterns. What stays here is what needs the store: resolving ids and host-side Transfers.
    pub const HipSession = struct {
        hb: *HipBackend,
        host: TensorStore,
        native: *c.aionhip_session,
        records: std.ArrayListUnmanaged(c.aionhip_step) = .{},

        pub fn create(hb: *HipBackend, store: TensorStore) tensor_store.StoreError!*HipSession {
            var native: ?*c.aionhip_session = null;
            if (c.aionhip_session_create(hb.ctx, &native) != c.AIONHIP_OK) return error.OutOfMemory;
            const s = hb.allocator.create(HipSession) catch {
                c.aionhip_session_destroy(native.?);
                return error.OutOfMemory;
            };
            s.* = .{ .hb = hb, .host = store, .native = native.? };
            return s;
        }

        fn execute(p: *anyopaque, prog: *const executable.ExecutableProgram) ExecuteProgramError!void {
            const s: *HipSession = @ptrCast(@alignCast(p));
            // a program carries the placement it was compiled for (backend/gpu/backend.zig:551-560)
            if (prog.target.kind != .hip) return BackendError.Unsupported;
            s.records.clearRetainingCapacity();
            for (prog.steps) |placed| {
                switch (placed.op) {
                    // a Transfer touches host storage under the store's access tokens: run what has gathered, then copy
                    .Transfer => |t| {
                        try s.flush();
                        try s.runTransfer(t);
                    },
                    else => s.records.append(s.hb.allocator, try s.record(prog, placed.op)) catch return tensor_store.StoreError.OutOfMemory,
                }
            }
            try s.flush();
        }
        fn flush(s: *HipSession) ExecuteProgramError!void {
            if (s.records.items.len == 0) return;
            defer s.records.clearRetainingCapacity();
            try check(c.aionhip_session_execute(s.native, s.records.items.ptr, s.records.items.len));
        }
        /// Wait for the stream, then drop what may retain tensor backings: the re-laid weights and the
        /// bf16 copies the context made of them. Called only before storage eviction (backend.zig:36-38).
        fn retireResources(p: *anyopaque) void {
            const s: *HipSession = @ptrCast(@alignCast(p));
            _ = c.aionhip_session_retire(s.native);
        }
        fn deinitSession(p: *anyopaque) void {
            const s: *HipSession = @ptrCast(@alignCast(p));
            c.aionhip_session_destroy(s.native);
            s.records.deinit(s.hb.allocator);
            s.hb.allocator.destroy(s);
        }
        const session_vtable = Session.VTable{ .execute = execute, .retireResources = retireResources, .deinit = deinitSession };

        fn addr(s: *HipSession, id: TensorId) ExecuteProgramError!u64 {
            const ref = (try s.host.deviceChunk(id, 0)) orelse return BackendError.InvalidArgument;
            return ref.handle;
        }

        /// What the store answers for one tensor id, as the library wants it. A tensor in one of the program's shared
        /// workspace slots (runtime/executable.zig:624-636) that is not a program output is dead after its last reader:
        /// the library may then fold the step that writes it into its consumer.
        fn tensorRef(s: *HipSession, prog: *const executable.ExecutableProgram, id: TensorId) ExecuteProgramError!c.aionhip_tensor_ref {
            const m = try s.host.meta(id);
            var t: c.aionhip_tensor_ref = std.mem.zeroes(c.aionhip_tensor_ref);
            if (m.rank > c.AIONHIP_MAX_RANK) return BackendError.Unsupported;
            t.handle = try s.addr(id);
            t.dtype = @intFromEnum(m.dtype);
            t.rank = m.rank;
            for (0..m.rank) |d| t.shape[d] = m.shape[d];
            if (s.host.sequenceCachePolicyInfo(id).kind == .rolling) t.flags |= c.AIONHIP_TENSOR_ROLLING;
            if (inWorkspace(prog, id)) t.flags |= c.AIONHIP_TENSOR_WORKSPACE;
            return t;
        }
        fn optRef(s: *HipSession, prog: *const executable.ExecutableProgram, id: ?TensorId) ExecuteProgramError!c.aionhip_tensor_ref {
            return if (id) |t| try s.tensorRef(prog, t) else std.mem.zeroes(c.aionhip_tensor_ref);
        }
        fn inWorkspace(prog: *const executable.ExecutableProgram, id: TensorId) bool {
            for (prog.outputs) |o| if (o == id) return false;
            for (prog.workspace_slots) |slot| {
                for (slot.members) |m| if (m == id) return true;
            }
            return false;
        }

        /// One step of a validated program as a record: `tag` is the Step union's own tag (declaration order,
        /// runtime/executable.zig:302-345), operands by role as include/aion_hip.h lists them. Tags the device does
        /// not run are passed on as they are: the library answers Unsupported for the list before it launches
        /// anything, and the compiler keeps such steps on the CPU (backend/backend.zig:85-107).
        fn record(s: *HipSession, prog: *const executable.ExecutableProgram, step: executable.Step) ExecuteProgramError!c.aionhip_step {
            var r: c.aionhip_step = std.mem.zeroes(c.aionhip_step);
            r.tag = @intFromEnum(std.meta.activeTag(step));
            switch (step) {
                .MatMul => |m| {
                    r.out = try s.tensorRef(prog, m.c);
                    r.in[0] = try s.tensorRef(prog, m.a);
                    r.in[1] = try s.tensorRef(prog, m.b);
                    r.alpha = m.alpha;
                    r.beta = m.beta;
                },
                .MatMulNT => |m| {
                    r.out = try s.tensorRef(prog, m.c);
                    r.in[0] = try s.tensorRef(prog, m.a);
                    r.in[1] = try s.tensorRef(prog, m.b);
                    r.alpha = m.alpha;
                    r.beta = m.beta;
                },
                .ElemwiseBinary => |e| {
                    r.out = try s.tensorRef(prog, e.out);
                    r.in[0] = try s.tensorRef(prog, e.a);
                    r.in[1] = try s.tensorRef(prog, e.b);
                    r.op = @intFromEnum(e.op);
                    r.act = @intFromEnum(e.act);
                    r.broadcast = @intFromEnum(e.broadcast.kind);
                },
                .Unary => |u| {
                    r.out = try s.tensorRef(prog, u.out);
                    r.in[0] = try s.tensorRef(prog, u.a);
                    r.op = @intFromEnum(u.op);
                },
                .RMSNorm => |n| {
                    r.out = try s.tensorRef(prog, n.out);
                    r.in[0] = try s.tensorRef(prog, n.x);
                    r.in[1] = try s.tensorRef(prog, n.gamma);
                    r.in[2] = try s.tensorRef(prog, n.beta);
                    r.in[3] = try s.optRef(prog, n.residual);
                    r.eps = n.eps;
                },
                .Attention => |a| {
                    r.out = try s.tensorRef(prog, a.out);
                    r.in[0] = try s.tensorRef(prog, a.q);
                    r.in[1] = try s.tensorRef(prog, a.k);
                    r.in[2] = try s.tensorRef(prog, a.v);
                    r.in[3] = try s.optRef(prog, a.query_positions);
                    r.in[4] = try s.optRef(prog, a.kv_lengths);
                    r.scale = a.scale;
                    r.soft_cap = a.attn_logits_soft_cap;
                    r.window_left = a.window.left;
                    r.window_right = a.window.right;
                    r.window_chunk = a.window.chunk;
                },
                .ArgMax => |a| {
                    r.out = try s.tensorRef(prog, a.out);
                    r.in[0] = try s.tensorRef(prog, a.a);
                    r.axis = @intCast(a.axis);
                },
                .Copy => |k| {
                    r.out = try s.tensorRef(prog, k.dst);
                    r.in[0] = try s.tensorRef(prog, k.src);
                },
                .GatherRows => |g| {
                    r.out = try s.tensorRef(prog, g.out);
                    r.in[0] = try s.tensorRef(prog, g.table);
                    r.in[1] = try s.tensorRef(prog, g.indices);
                },
                .Gather => |g| {
                    r.out = try s.tensorRef(prog, g.out);
                    r.in[0] = try s.tensorRef(prog, g.data);
                    r.in[1] = try s.tensorRef(prog, g.indices);
                    r.axis = @intCast(g.axis);
                    r.batch_dims = @intCast(g.batch_dims);
                },
                .RoPE1D => |p| {
                    r.out = try s.tensorRef(prog, p.out);
                    r.in[0] = try s.tensorRef(prog, p.x);
                    r.in[1] = try s.tensorRef(prog, p.positions);
                    r.rope_base = p.base_frequency;
                    r.rope_scale = p.scale_factor;
                    r.rope_proportion = p.rope_proportion;
                },
                .SequenceAppend => |a| {
                    r.out = try s.tensorRef(prog, a.cache);
                    r.in[0] = try s.tensorRef(prog, a.new_kv);
                    r.in[1] = try s.tensorRef(prog, a.end_index);
                },
                .Cast => |k| {
                    r.out = try s.tensorRef(prog, k.out);
                    r.in[0] = try s.tensorRef(prog, k.x);
                },
                // no operands needed: the tag alone makes the library answer Unsupported for the list
                else => {},
            }
            return r;
        }

        /// Host <-> device copy placed by the compiler (backend/gpu/backend.zig:416-457). Both copies are ordered on
        /// the context's stream; the device-to-host one returns when the bytes have arrived, which makes it the
        /// program's synchronisation point.
        fn runTransfer(s: *HipSession, t: executable.StepTransfer) ExecuteProgramError!void {
            const ctx = s.hb.ctx;
            const to_host = t.source.kind == .hip and t.destination.kind == .cpu;
            const to_device = t.source.kind == .cpu and t.destination.kind == .hip;
            if (!to_host and !to_device) return BackendError.Unsupported;
            const sm = s.host.meta(t.src) catch return BackendError.ExecutionFailed;
            const dmeta = s.host.meta(t.dst) catch return BackendError.ExecutionFailed;
            if (sm.dtype != dmeta.dtype) return BackendError.ExecutionFailed;
            if (to_host) {
                const host = s.host.acquireMut(t.dst) catch return BackendError.ExecutionFailed;
                defer s.host.releaseMut(host.token);
                try check(c.aionhip_d2h(ctx, host.bytes.ptr, try s.addr(t.src), 0, host.bytes.len));
            } else {
                const host = s.host.acquireConst(t.src) catch return BackendError.ExecutionFailed;
                defer s.host.releaseConst(host.token);
                try check(c.aionhip_h2d(ctx, try s.addr(t.dst), 0, host.bytes.ptr, host.bytes.len));
            }
        }
    };

    // What aionhip_session_execute folds (each gives the separate steps' results bit for bit; AIONHIP_FUSE_* of
    // aionhip_session_set_fusion switches them off):
    //   RMSNorm, MatMul x3 (q,k,v), RoPE1D x2, Cast f16 x2, SequenceAppend x2, one token -> aionhip_step_rmsnorm_qkv_rope_append
    //   RMSNorm, MatMul x2 (gate, up), gate(gelu), MatMul (down), one row              -> aionhip_step_rmsnorm_geglu_matmul
    //   RMSNorm, MatMul(s)                                                             -> aionhip_step_rmsnorm_matmul
    //   gate(gelu), MatMul                                                             -> aionhip_step_gate_matmul
    //   Cast f32->f16, SequenceAppend                                                  -> aionhip_step_append_f16
    //   MatMul(s) sharing one A                                                        -> aionhip_step_matmul_batch
    //   MatMul, add in place (x = x + t), alone or behind the patterns above           -> the matmul with C = x, beta = 1
    //   RMSNorm x3 per head (q,k,v), RoPE1D x2, Cast f16 x2, SequenceAppend x2         -> aionhip_step_headnorm_rope_append
    //   RoPE1D x2, Cast f16 x2, SequenceAppend x2 (linear caches)                      -> aionhip_step_rope_append
    // A whole decode program (no If/Loop, no Transfer) may be recorded once between aionhip_program_begin/_end around
    // aionhip_session_execute and replayed with aionhip_program_execute while aionhip_program_is_current holds (replay
    // precedent: backend/gpu/frame.zig:77-86).
};
