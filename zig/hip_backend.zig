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
const TensorMeta = tensor_store.TensorMeta;

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

    /// The owner calls this; the vtable's `deinit` is a no-op like backend/gpu/backend.zig:675-678.
    pub fn deinit(self: *HipBackend) void {
        self.dropWeights();
        self.weights.deinit();
        c.aionhip_destroy(self.ctx);
    }

    fn dropWeights(self: *HipBackend) void {
        var it = self.weights.valueIterator();
        while (it.next()) |w| c.aionhip_weight_free(self.ctx, w.*);
        self.weights.clearRetainingCapacity();
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
        const s = self.allocator.create(HipSession) catch return error.OutOfMemory;
        s.* = .{ .hb = self, .host = store };
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

    /// A session bound to one placed tensor store (backend/gpu/backend.zig:206-270). Tensors the store placed on
    /// this device answer `deviceChunk` (runtime/tensor_store.zig:150-201) with one chunk: the whole buffer.
    pub const HipSession = struct {
        hb: *HipBackend,
        host: TensorStore,

        fn execute(p: *anyopaque, prog: *const executable.ExecutableProgram) ExecuteProgramError!void {
            const s: *HipSession = @ptrCast(@alignCast(p));
            // a program carries the placement it was compiled for (backend/gpu/backend.zig:551-560)
            if (prog.target.kind != .hip) return BackendError.Unsupported;
            for (prog.steps) |placed| try s.dispatchStep(placed.op);
        }
        /// Wait for the stream, then drop what may retain tensor backings: the re-laid weights and the
        /// bf16 copies the context made of them. Called only before storage eviction (backend.zig:36-38).
        fn retireResources(p: *anyopaque) void {
            const s: *HipSession = @ptrCast(@alignCast(p));
            _ = c.aionhip_sync(s.hb.ctx);
            s.hb.dropWeights();
        }
        fn deinitSession(p: *anyopaque) void {
            const s: *HipSession = @ptrCast(@alignCast(p));
            s.hb.allocator.destroy(s);
        }
        const session_vtable = Session.VTable{ .execute = execute, .retireResources = retireResources, .deinit = deinitSession };

        fn addr(s: *HipSession, id: TensorId) ExecuteProgramError!u64 {
            const ref = (try s.host.deviceChunk(id, 0)) orelse return BackendError.InvalidArgument;
            return ref.handle;
        }
        fn optAddr(s: *HipSession, id: ?TensorId) ExecuteProgramError!u64 {
            return if (id) |t| try s.addr(t) else 0;
        }

        // weights: re-laid at first use, straight from the packed blocks already on the device
        fn weightFor(s: *HipSession, id: TensorId, layout: c_int) ExecuteProgramError!*c.aionhip_weight {
            const hb = s.hb;
            const meta = try s.host.meta(id);
            const handle = try s.addr(id);
            if (hb.weights.get(handle)) |w| return w;
            const n = if (layout == c.AIONHIP_ROWS_NK) meta.shape[0] else meta.shape[1];
            const k = if (layout == c.AIONHIP_ROWS_NK) meta.shape[1] else meta.shape[0];
            var w: ?*c.aionhip_weight = null;
            try check(c.aionhip_weight_from_device(hb.ctx, @intFromEnum(meta.dtype), layout, n, k, 0, handle, &w));
            hb.weights.put(handle, w.?) catch return tensor_store.StoreError.OutOfMemory;
            return w.?;
        }

        /// One step of a validated program (the reduced twin of backend/gpu/backend.zig:459-548): the steps of
        /// a quantized decoder; every other tag is Unsupported and the compiler keeps it on the CPU.
        fn dispatchStep(s: *HipSession, step: executable.Step) ExecuteProgramError!void {
            const ctx = s.hb.ctx;
            switch (step) {
                .MatMul => |m| {
                    const w = try s.weightFor(m.b, c.AIONHIP_KMAJOR_KN);
                    try check(c.aionhip_step_matmul(ctx, w, rowsOf(try s.host.meta(m.a)), try s.addr(m.a), 0, try s.addr(m.c), 0, m.alpha, m.beta));
                },
                .MatMulNT => |m| {
                    const w = try s.weightFor(m.b, c.AIONHIP_ROWS_NK);
                    try check(c.aionhip_step_matmul_nt(ctx, w, rowsOf(try s.host.meta(m.a)), try s.addr(m.a), 0, try s.addr(m.c), 0, m.alpha, m.beta));
                },
                .Attention => |a| {
                    const qm = try s.host.meta(a.q);
                    const km = try s.host.meta(a.k);
                    const vm = try s.host.meta(a.v);
                    var p: c.aionhip_attention = std.mem.zeroes(c.aionhip_attention);
                    p.out = try s.addr(a.out);
                    p.q = try s.addr(a.q);
                    p.k = try s.addr(a.k);
                    p.v = try s.addr(a.v);
                    p.query_positions = try s.optAddr(a.query_positions);
                    p.kv_lengths = try s.optAddr(a.kv_lengths);
                    p.batch = qm.shape[0]; p.l_q = qm.shape[1]; p.h_q = qm.shape[2]; p.d_k = qm.shape[3];
                    p.t_kv = km.shape[1]; p.h_kv = km.shape[2]; p.d_v = vm.shape[3];
                    p.q_dtype = @intFromEnum(qm.dtype); p.kv_dtype = @intFromEnum(km.dtype);
                    p.scale = a.scale; p.attn_logits_soft_cap = a.attn_logits_soft_cap;
                    p.window_left = a.window.left; p.window_right = a.window.right; p.window_chunk = a.window.chunk;
                    // a rolling sequence cache reads key t from row t % capacity (cpu/exec/attention.zig:1537-1546)
                    p.rolling = if (s.host.sequenceCachePolicyInfo(a.k).kind == .rolling) 1 else 0;
                    try check(c.aionhip_step_attention(ctx, &p));
                },
                .RMSNorm => |n| {
                    const cols = elemCount(try s.host.meta(n.gamma));
                    try check(c.aionhip_step_rmsnorm(ctx, try s.addr(n.out), try s.addr(n.x), try s.addr(n.gamma), try s.addr(n.beta),
                        try s.optAddr(n.residual), elemCount(try s.host.meta(n.out)) / cols, cols, n.eps));
                },
                .RoPE1D => |r| {
                    const m = try s.host.meta(r.out);
                    try check(c.aionhip_step_rope(ctx, try s.addr(r.out), try s.addr(r.x), try s.addr(r.positions),
                        m.shape[0], m.shape[1], m.shape[2], m.shape[3], r.base_frequency, r.scale_factor, r.rope_proportion));
                },
                .ArgMax => |a| {
                    const m = try s.host.meta(a.a);
                    if (a.axis + 1 != m.rank) return BackendError.Unsupported;
                    const n = m.shape[m.rank - 1];
                    try check(c.aionhip_step_argmax(ctx, try s.addr(a.out), try s.addr(a.a), elemCount(m) / n, n));
                },
                .ElemwiseBinary => |e| {
                    const am = try s.host.meta(e.a);
                    const n = elemCount(try s.host.meta(e.out));
                    if (am.dtype == .i32) {
                        // the decode counters (position + 1): same-shape i32 add only
                        if (e.op != .add or e.broadcast.kind != .identical) return BackendError.Unsupported;
                        return check(c.aionhip_step_add_i32(ctx, try s.addr(e.out), try s.addr(e.a), try s.addr(e.b), n));
                    }
                    if (e.op == .gate) {
                        // gate(a, b) = act(a) * b (backend/types.zig:105-109); the device kernel is the gelu form
                        if (e.act != .gelu or e.broadcast.kind != .identical) return BackendError.Unsupported;
                        return check(c.aionhip_step_gate_gelu(ctx, try s.addr(e.out), try s.addr(e.a), try s.addr(e.b), n));
                    }
                    // add/sub/mul/div carry ElemwiseBinaryOp's own ids (backend/types.zig:92-96) across the ABI;
                    // b may be the same shape, one element or a contiguous suffix of a's shape
                    const op: c_int = switch (e.op) {
                        .add, .sub, .mul, .div => @intFromEnum(e.op),
                        else => return BackendError.Unsupported,
                    };
                    const nb: usize = switch (e.broadcast.kind) {
                        .identical => n,
                        .scalar_b => 1,
                        .contiguous_suffix_b => elemCount(try s.host.meta(e.b)),
                        else => return BackendError.Unsupported,
                    };
                    try check(c.aionhip_step_binary(ctx, op, try s.addr(e.out), try s.addr(e.a), try s.addr(e.b), n, nb));
                },
                .Unary => |u| {
                    // UnaryOp's ids are the ABI's (backend/types.zig:119-128); log answers AIONHIP_UNSUPPORTED
                    try check(c.aionhip_step_unary(ctx, @intFromEnum(u.op), try s.addr(u.out), try s.addr(u.a), elemCount(try s.host.meta(u.out))));
                },
                .Gather => |g| {
                    // embedding lookup: rows of a [V, D] table (f32, or q8_0 blocked along D) by i32 ids
                    const tm = try s.host.meta(g.data);
                    if (g.axis != 0 or g.batch_dims != 0 or tm.rank != 2) return BackendError.Unsupported;
                    try check(c.aionhip_step_gather_rows(ctx, @intFromEnum(tm.dtype), try s.addr(g.out), try s.addr(g.data), try s.addr(g.indices),
                        elemCount(try s.host.meta(g.indices)), tm.shape[1], tm.shape[0]));
                },
                .GatherRows => |g| {
                    const tm = try s.host.meta(g.table);
                    try check(c.aionhip_step_gather_rows(ctx, @intFromEnum(tm.dtype), try s.addr(g.out), try s.addr(g.table), try s.addr(g.indices),
                        elemCount(try s.host.meta(g.indices)), tm.shape[1], tm.shape[0]));
                },
                .Cast => |k| {
                    const xm = try s.host.meta(k.x);
                    if (xm.dtype != .f32 or k.to_dtype != .f16) return BackendError.Unsupported;
                    try check(c.aionhip_step_cast_f32_f16(ctx, try s.addr(k.out), try s.addr(k.x), elemCount(xm)));
                },
                .SequenceAppend => |a| {
                    // cache [B, T, H, D] and rows [B, S, H, D] of one element type (cpu/exec/sequence_append.zig:29-31)
                    const cm = try s.host.meta(a.cache);
                    const nm = try s.host.meta(a.new_kv);
                    const rolling: c_int = if (s.host.sequenceCachePolicyInfo(a.cache).kind == .rolling) 1 else 0;
                    try check(c.aionhip_step_sequence_append(ctx, @intFromEnum(cm.dtype), try s.addr(a.cache), try s.addr(a.new_kv), try s.addr(a.end_index),
                        cm.shape[0], nm.shape[1], cm.shape[1], cm.shape[2] * cm.shape[3], rolling));
                },
                .Copy => |k| {
                    const m = try s.host.meta(k.dst);
                    try check(c.aionhip_d2d(ctx, try s.addr(k.dst), 0, try s.addr(k.src), 0, byteCount(m)));
                },
                .Transfer => |t| try s.runTransfer(t),
                else => return BackendError.Unsupported,
            }
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

    // Optional launch-saving pattern matches over consecutive steps of a decode program; each gives the results of
    // the separate steps bit for bit, and a maintainer falls back to those on AIONHIP_UNSUPPORTED:
    //   RMSNorm, MatMul x3 (q,k,v), RoPE1D x2, Cast f16 x2, SequenceAppend x2 -> aionhip_step_rmsnorm_qkv_rope_append
    //   RMSNorm x3 (per head, q,k,v), RoPE1D x2, Cast f16 x2, SequenceAppend x2 -> aionhip_step_headnorm_rope_append
    //   RMSNorm, MatMul x2 (gate, up), gate(gelu), MatMul (down)             -> aionhip_step_rmsnorm_geglu_matmul
    //   RMSNorm, MatMul(s)                                                   -> aionhip_step_rmsnorm_matmul
    //   gate(gelu), MatMul                                                   -> aionhip_step_gate_matmul
    //   MatMul(s) sharing one A                                              -> aionhip_step_matmul_batch
    //   Cast f32->f16 feeding only a SequenceAppend                          -> aionhip_step_append_f16
    // A whole decode program (no If/Loop) may be recorded once between aionhip_program_begin/_end and replayed with
    // aionhip_program_execute while aionhip_program_is_current holds (replay precedent: backend/gpu/frame.zig:77-86).

    fn rowsOf(m: TensorMeta) usize {
        var r: usize = 1;
        for (0..m.rank - 1) |d| r *= m.shape[d];
        return r;
    }
    fn elemCount(m: TensorMeta) usize {
        var r: usize = 1;
        for (0..m.rank) |d| r *= m.shape[d];
        return r;
    }
    fn byteCount(m: TensorMeta) usize {
        const info = m.dtype.info();
        return elemCount(m) / info.block_elems * info.block_bytes;
    }
};
