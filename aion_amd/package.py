"""Runs a decoder-style `.aion` package on the HIP backend: the graph's nodes, in file order, become the
backend's steps (the subset of aion's lowering `graph/program/compiler.zig:1052-1153` that a quantized decoder
needs). One device buffer per produced value; views alias their source; KV caches are the io-aliased inputs and
stay on the device between runs (roles from the package's `input_roles`, `storage/aion_file/types.zig:164-198`).

Mapping (node -> step), with the three places where consecutive nodes become one step because the step exists
in that form only:
  Gather axis 0                       -> aionhip_step_gather_rows
  RMSNorm (x, gamma, beta)            -> aionhip_step_rmsnorm
  MatMul (a, W)                       -> aionhip_step_matmul; W is a q4_0 [K,N] quant_axis 0 initializer, or
                                         ViewTranspose2D of a q8_0 [N,K] quant_axis 1 initializer (aion lowers that
                                         pair to MatMulNT, graph/program/matmul_rows.zig:1-13)
  ViewReshape / Squeeze / Unsqueeze   -> alias
  RoPE1D                              -> aionhip_step_rope
  Cast f32->f16 + SequenceAppend      -> aionhip_step_append_f16 (the cast is materialised only if something
                                         else reads it)
  Attention                           -> aionhip_step_attention
  Unary gelu + ElemwiseBinary mul     -> aionhip_step_gate_gelu (aion's own `gate` step fusion, graph/opt/fuse_steps.zig)
  ElemwiseBinary add                  -> aionhip_step_add
  ArgMax axis -1                      -> aionhip_step_argmax
Anything else raises Unsupported: aion's placement pass keeps such ops on the CPU backend.
"""
import numpy as np

from . import backend as be
from .aion_file import PackageError

_ELEM = {"f32": 4, "f16": 2, "i32": 4, "i8": 1}


class Unsupported(RuntimeError):
    pass


class _Val:
    __slots__ = ("kind", "buf", "shape", "dtype", "extra", "owned")

    def __init__(self, kind, buf, shape, dtype, extra=None, owned=False):
        self.kind, self.buf, self.shape, self.dtype, self.extra, self.owned = kind, buf, tuple(shape), dtype, extra, owned


def _count(shape):
    n = 1
    for d in shape:
        n *= int(d)
    return n


class PackageRunner:
    def __init__(self, gpu, pkg, capacity, capacity_symbol="ctx", tokens_symbol="seq"):
        self.gpu, self.pkg, self.capacity = gpu, pkg, int(capacity)
        self.sym_ctx, self.sym_seq = capacity_symbol, tokens_symbol
        self.pos = 0
        self.consts = {}            # value id -> _Val of an uploaded initializer
        self.caches = {}            # input index -> device buffer
        self.consumers = {}
        for n in pkg.nodes:
            for i in n.inputs:
                self.consumers[i] = self.consumers.get(i, 0) + 1
        for _name, vid in pkg.outputs:
            self.consumers[vid] = self.consumers.get(vid, 0) + 1
        self.producer = {n.output: n for n in pkg.nodes}
        self.roles = {}
        for idx, (_name, vid) in enumerate(pkg.inputs):
            role = pkg.role_of_input(idx)
            if role is None:
                raise Unsupported("input %d has no role: this runner feeds inputs by role" % idx)
            self.roles[vid] = (idx, role)
            if role.kind == "sequence_cache":
                shape = pkg.shape_of(vid, {self.sym_ctx: self.capacity, self.sym_seq: 1})
                if pkg.values[vid].dtype != "f16":
                    raise Unsupported("sequence cache of dtype %s" % pkg.values[vid].dtype)
                self.caches[idx] = gpu.zeros(_count(shape) * 2)

    # ---- initializers
    def _const(self, vid, transposed=False):
        key = (vid, transposed)
        if key in self.consts:
            return self.consts[key]
        v = self.pkg.values[vid]
        t = self.pkg.tensors[v.initializer]
        shape = self.pkg.shape_of(vid, {})
        if t.quantized:
            if len(shape) != 2:
                raise Unsupported("quantized initializer of rank %d" % len(shape))
            if t.scheme == "q4_0" and t.quant_axis == 0 and not transposed:
                k, n = shape
                w = self.gpu.upload_weight(be.Q4_0, be.KMAJOR_KN, n, k, np.asarray(t.data))
            elif t.scheme == "q8_0" and t.quant_axis == 0 and not transposed:
                k, n = shape
                w = self.gpu.upload_weight(be.Q8_0, be.KMAJOR_KN, n, k, np.asarray(t.data))
            elif t.scheme == "q8_0" and t.quant_axis == 1 and transposed:
                n, k = shape
                w = self.gpu.upload_weight(be.Q8_0, be.ROWS_NK, n, k, np.asarray(t.data))
            else:
                raise Unsupported("%s initializer with quant_axis %d%s as a matmul operand" %
                                  (t.scheme, t.quant_axis, " under a transpose" if transposed else ""))
            val = _Val("weight", w, shape, t.scheme)
        else:
            if transposed:
                raise Unsupported("transpose of a plain initializer")
            if _count(shape) * _ELEM[t.dtype] != t.data.size:
                raise PackageError("InvalidFormat", "initializer payload does not match its shape")
            val = _Val("dev", self.gpu.upload(np.asarray(t.data)), shape, t.dtype)
        self.consts[key] = val
        return val

    # ---- one run
    def run(self, tokens, want=("next_token",)):
        """Feeds `tokens` (int32 [S]) at positions pos..pos+S-1, runs the graph, advances pos. Returns the
        requested outputs (by signature name) as numpy arrays."""
        g, pkg = self.gpu, self.pkg
        tokens = np.ascontiguousarray(tokens, np.int32).reshape(-1)
        s = tokens.size
        if self.pos + s > self.capacity:
            raise ValueError("the run exceeds the cache capacity")
        sym = {self.sym_seq: s, self.sym_ctx: self.capacity}
        vals, temps = {}, []

        def new(shape, dtype):
            buf = g.alloc(max(_count(shape) * _ELEM[dtype], 4))
            temps.append(buf)
            return buf

        for vid, (idx, role) in self.roles.items():
            shape = pkg.shape_of(vid, sym)
            if role.kind == "tokens":
                arr = tokens
            elif role.kind == "positions":
                arr = np.arange(self.pos, self.pos + s, dtype=np.int32)
            elif role.kind == "cache_write_index":
                arr = np.array([self.pos], np.int32)
            elif role.kind == "cache_visible_end":
                arr = np.array([self.pos + s], np.int32)
            elif role.kind == "sequence_cache":
                vals[vid] = _Val("dev", self.caches[idx], shape, "f16")
                continue
            else:
                raise Unsupported("input role %s" % role.kind)
            if _count(shape) != arr.size:
                raise PackageError("InvalidArgument", "input %d: shape %s for %d elements" % (idx, shape, arr.size))
            buf = g.upload(arr)
            temps.append(buf)
            vals[vid] = _Val("dev", buf, shape, "i32")

        def get(vid):
            """The device value of `vid`, materialising a pending cast."""
            if vid not in vals:
                if pkg.values[vid].source != "initializer":
                    raise PackageError("InvalidFormat", "value %d is read before it is produced" % vid)
                vals[vid] = self._const(vid)
            v = vals[vid]
            if v.kind == "cast":
                src = get(v.extra)
                out = new(v.shape, "f16")
                g.step_cast_f32_f16(out, src.buf, _count(v.shape))
                v = vals[vid] = _Val("dev", out, v.shape, "f16")
            elif v.kind == "gelu":
                raise Unsupported("a gelu that does not feed a multiply (aion's gate step)")
            return v

        try:
            for n in pkg.nodes:
                shape = pkg.shape_of(n.output, sym)
                dtype = pkg.values[n.output].dtype
                op, a = n.op, n.attrs
                if op == "Gather":
                    table, ids = get(n.inputs[0]), get(n.inputs[1])
                    if a["axis"] != 0 or a["batch_dims"] != 0 or len(table.shape) != 2 or table.dtype != "f32":
                        raise Unsupported("Gather other than rows of an f32 table")
                    out = new(shape, "f32")
                    g.step_gather_rows(be.F32, out, table.buf, ids.buf, _count(ids.shape), table.shape[1], table.shape[0])
                    vals[n.output] = _Val("dev", out, shape, "f32")
                elif op == "RMSNorm":
                    x, gamma, beta = get(n.inputs[0]), get(n.inputs[1]), get(n.inputs[2])
                    cols = 1
                    for t in a["normalized_shape"]:
                        cols *= pkg.dim_term(t, sym)
                    if cols != x.shape[-1]:
                        raise Unsupported("RMSNorm over more than the last axis")
                    out = new(shape, "f32")
                    g.step_rmsnorm(out, x.buf, gamma.buf, _count(x.shape) // cols, cols, a["eps"], beta=beta.buf)
                    vals[n.output] = _Val("dev", out, shape, "f32")
                elif op == "ViewTranspose2D":
                    src = n.inputs[0]
                    if pkg.values[src].source != "initializer":
                        raise Unsupported("ViewTranspose2D of a computed value")
                    vals[n.output] = self._const(src, transposed=True)
                elif op == "MatMul":
                    x = get(n.inputs[0])
                    w = vals[n.inputs[1]] if n.inputs[1] in vals else self._const(n.inputs[1])
                    if w.kind != "weight":
                        raise Unsupported("MatMul whose right operand is not a quantized weight")
                    if a["beta"] != 0.0:
                        raise Unsupported("MatMul with beta != 0 in a package")
                    out = new(shape, "f32")
                    g.step_matmul(w.buf, x.buf, _count(x.shape[:-1]), out, alpha=a["alpha"])
                    vals[n.output] = _Val("dev", out, shape, "f32")
                elif op in ("ViewReshape", "ViewSqueeze", "ViewUnsqueeze"):
                    x = get(n.inputs[0])
                    if _count(shape) != _count(x.shape):
                        raise PackageError("InvalidFormat", "view changes the element count")
                    vals[n.output] = _Val("dev", x.buf, shape, x.dtype)
                elif op == "RoPE1D":
                    x, pos = get(n.inputs[0]), get(n.inputs[1])
                    if len(x.shape) != 4:
                        raise Unsupported("RoPE1D on rank %d" % len(x.shape))
                    out = new(shape, "f32")
                    g.step_rope(out, x.buf, pos.buf, x.shape[0], x.shape[1], x.shape[2], x.shape[3], base=a["base_frequency"],
                                scale_factor=a["scale_factor"], proportion=a["rope_proportion"])
                    vals[n.output] = _Val("dev", out, shape, "f32")
                elif op == "Cast":
                    if a["to_dtype"] != "f16" or pkg.values[n.inputs[0]].dtype != "f32":
                        raise Unsupported("Cast other than f32 -> f16")
                    vals[n.output] = _Val("cast", None, shape, "f16", extra=n.inputs[0])
                elif op == "SequenceAppend":
                    cache, widx = get(n.inputs[0]), get(n.inputs[2])
                    newv = vals.get(n.inputs[1])
                    if newv is None or newv.kind != "cast":
                        raise Unsupported("SequenceAppend whose new rows are not a Cast f32 -> f16")
                    src = get(newv.extra)
                    bsz, t_cap = cache.shape[0], cache.shape[1]
                    g.step_append_f16(cache.buf, src.buf, widx.buf, bsz, newv.shape[1], t_cap, _count(cache.shape[2:]))
                    vals[n.output] = _Val("dev", cache.buf, shape, "f16")
                elif op == "Attention":
                    q, k, v = get(n.inputs[0]), get(n.inputs[1]), get(n.inputs[2])
                    rest = list(n.inputs[3:])
                    pos = get(rest.pop(0)) if a["has_query_positions"] else None
                    lens = get(rest.pop(0)) if a["has_kv_lengths"] else None
                    w = a["window"]
                    out = new(shape, "f32")
                    dts = {"f32": be.F32, "f16": be.F16}
                    g.step_attention(out, q.buf, k.buf, v.buf,
                                     (q.shape[0], q.shape[1], k.shape[1], q.shape[2], k.shape[2], q.shape[3], v.shape[3]), a["scale"],
                                     q_dtype=dts[q.dtype], kv_dtype=dts[k.dtype], window=(w["left"], w["right"], w["chunk"]),
                                     soft_cap=a["soft_cap"], query_positions=pos.buf if pos else None,
                                     kv_lengths=lens.buf if lens else None)
                    vals[n.output] = _Val("dev", out, shape, "f32")
                elif op == "Unary":
                    if a["op"] != "gelu":
                        raise Unsupported("Unary %s" % a["op"])
                    vals[n.output] = _Val("gelu", None, shape, "f32", extra=n.inputs[0])
                elif op == "ElemwiseBinary":
                    if a["op"] == "add":
                        x, y = get(n.inputs[0]), get(n.inputs[1])
                        if x.shape != y.shape:
                            raise Unsupported("broadcasting add")
                        out = new(shape, "f32")
                        g.step_add(out, x.buf, y.buf, _count(shape))
                    elif a["op"] == "mul":
                        lhs = vals.get(n.inputs[0])
                        if lhs is None or lhs.kind != "gelu":
                            raise Unsupported("a multiply that is not gelu(gate) * up")
                        gate, up = get(lhs.extra), get(n.inputs[1])
                        out = new(shape, "f32")
                        g.step_gate_gelu(out, gate.buf, up.buf, _count(shape))
                    else:
                        raise Unsupported("ElemwiseBinary %s" % a["op"])
                    vals[n.output] = _Val("dev", out, shape, "f32")
                elif op == "ArgMax":
                    x = get(n.inputs[0])
                    if a["axis"] not in (-1, len(x.shape) - 1):
                        raise Unsupported("ArgMax over an inner axis")
                    out = new(shape, "i32")
                    g.step_argmax(out, x.buf, _count(x.shape[:-1]), x.shape[-1])
                    vals[n.output] = _Val("dev", out, shape, "i32")
                else:
                    raise Unsupported("operation %s has no step on this backend" % op)

            result = {}
            for name, vid in pkg.outputs:
                if name in want:
                    v = get(vid)
                    result[name] = g.download(v.buf, {"f32": np.float32, "i32": np.int32, "f16": np.float16}[v.dtype], v.shape)
            g.sync()
        finally:
            for t in temps:
                t.free()
        self.pos += s
        return result

    def reset(self):
        self.pos = 0

    def close(self):
        for c in self.consts.values():
            c.buf.free()
        for b in self.caches.values():
            b.free()
        self.consts, self.caches = {}, {}
