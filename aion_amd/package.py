"""Runs a decoder-style `.aion` package on the HIP backend: the graph's nodes, in file order, become the
backend's steps (the subset of aion's lowering `graph/program/compiler.zig:1052-1153` that a quantized decoder
needs). One device buffer per produced value; views alias their source; KV caches are the io-aliased inputs and
stay on the device between runs (roles from the package's `input_roles`, `storage/aion_file/types.zig:164-198`).

A plan is built once per number of new tokens: buffers are allocated then, and a run only writes the inputs,
issues the plan's steps and reads the outputs back. For one new token the plan can be recorded as a program
(HIP graph) whose token, position, write index and visible end stay on the device (`begin_decode` / `decode_step`).

Mapping (node -> step). Consecutive nodes become one step where the step exists in that form only:
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

On top of that, the step-level fusions of aion's schedule (graph/opt/fuse_steps.zig, graph/program/matmul_rows.zig)
and this backend's optional fused steps, each found by walking the consumers of a node and applied only when every
intermediate value has no other reader:
  RMSNorm -> MatMul(s) on its output                          -> aionhip_step_rmsnorm_matmul
  gelu(gate) * up -> MatMul                                   -> aionhip_step_gate_matmul
  MatMul -> add(residual, .) whose residual is dead afterwards -> beta = 1 into the residual's buffer
  one new token: RMSNorm -> MatMul q,k,v -> reshape -> RoPE1D(q,k) -> Cast -> SequenceAppend(k,v)
                                                              -> aionhip_step_rmsnorm_qkv_rope_append
  one new token: RMSNorm -> MatMul gate,up -> gelu*up -> MatMul down -> add(residual, .)
                                                              -> aionhip_step_rmsnorm_geglu_matmul
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


_VIEWS = ("ViewReshape", "ViewSqueeze", "ViewUnsqueeze")
_OUT = 1 << 30          # "consumer index" of a graph output


class _Plan:
    def __init__(self):
        self.steps, self.buffers, self.inputs, self.outputs, self.values = [], [], {}, {}, {}


class PackageRunner:
    LOG_TOKENS = 4096                      # tokens decode_run leaves on the device between two read-backs

    def __init__(self, gpu, pkg, capacity, capacity_symbol="ctx", tokens_symbol="seq", fuse=True, growth=None, keep_residuals=False):
        """growth: None = the capacity is fixed and a run that needs more is an error. A dict with "numerator",
        "denominator" and optionally "max_capacity" = the sequence caches grow on the device when a run needs more
        rows, on the schedule of aion's session (api/loaded_model.zig:735-827: geometric steps, then a power of
        two and at least four times the old capacity, since every capacity is a set of plans of its own; rolling
        caches use the factor 2/1 and are re-placed row by row).
        keep_residuals: a residual add folded into a matmul's beta normally overwrites the residual in place, so that after a
        run only the last layer's residual stream is left on the device. True = the sum goes to a buffer of its own (one
        device copy of the residual first, then the same beta = 1 launch), which keeps every layer's input readable after
        the run through `plans[s].values` - for inspecting a fused schedule node by node, not for speed."""
        self.gpu, self.pkg, self.capacity, self.fuse = gpu, pkg, int(capacity), fuse
        self.keep_residuals = keep_residuals
        self.growth = growth
        self.cache_meta = {}        # input index -> (value id, retained history tokens, rows if the capacity is a constant else None)
        self.sym_ctx, self.sym_seq = capacity_symbol, tokens_symbol
        self.pos = 0
        self.consts = {}            # (value id, transposed) -> _Val of an uploaded initializer
        self.caches = {}            # input index -> device buffer
        self.plans = {}             # new tokens per run -> _Plan
        self.program = None
        self.one = None
        self.log = self.log_at = None      # device token log of decode_run and its counter
        self.uses = {}
        for i, n in enumerate(pkg.nodes):
            for v in n.inputs:
                self.uses.setdefault(v, []).append(i)
        for _name, vid in pkg.outputs:
            self.uses.setdefault(vid, []).append(_OUT)
        self.roles = {}
        self.all_rolling = all(r.retained_history_tokens for r in pkg.input_roles if r.kind == "sequence_cache") and \
            any(r.kind == "sequence_cache" for r in pkg.input_roles)
        for idx, (_name, vid) in enumerate(pkg.inputs):
            role = pkg.role_of_input(idx)
            if role is None:
                raise Unsupported("input %d has no role: this runner feeds inputs by role" % idx)
            self.roles[vid] = (idx, role)
            if role.kind == "sequence_cache":
                shape = pkg.shape_of(vid, {self.sym_ctx: self.capacity, self.sym_seq: 1})
                if pkg.values[vid].dtype != "f16":
                    raise Unsupported("sequence cache of dtype %s" % pkg.values[vid].dtype)
                if growth is not None and not (role.flags & 2) and not role.retained_history_tokens:
                    raise Unsupported("input %d does not allow growth (InputRoleFlags.allow_growable)" % idx)
                self.caches[idx] = gpu.zeros(_count(shape) * 2)
                self.cache_meta[idx] = (vid, int(role.retained_history_tokens), None if role.capacity_symbol != 0xFFFFFFFF else shape[1])

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
            elif t.scheme == "q8_0" and t.quant_axis == 1:
                # rows of 34-byte blocks as the file holds them: a Gather table (cpu/exec/gather.zig:60-87). The same
                # initializer under a ViewTranspose2D (a tied logits head) is uploaded a second time in the matmul layout.
                if shape[1] % 32:
                    raise Unsupported("a q8_0 gather table whose rows are not whole blocks")
                val = _Val("qtable", self.gpu.upload(np.asarray(t.data)), shape, "q8_0")
                self.consts[key] = val
                return val
            else:
                raise Unsupported("%s initializer with quant_axis %d%s as a matmul operand" %
                                  (t.scheme, t.quant_axis, " under a transpose" if transposed else ""))
            val = _Val("weight", w, shape, t.scheme)
        else:
            if _count(shape) * _ELEM[t.dtype] != t.data.size:
                raise PackageError("InvalidFormat", "initializer payload does not match its shape")
            if transposed:
                # MatMul over the transpose of a plain f32 [N,K] initializer is MatMulNT with an f32 B
                # (graph/program/compiler.zig:337-357, cpu/exec/matmul_nt.zig:100)
                if t.dtype != "f32" or len(shape) != 2:
                    raise Unsupported("transpose of a plain %s initializer of rank %d" % (t.dtype, len(shape)))
                n, k = shape
                w = self.gpu.upload_weight(be.F32, be.ROWS_NK, n, k, np.frombuffer(np.asarray(t.data), np.float32))
                val = _Val("weight", w, shape, "f32")
            else:
                val = _Val("dev", self.gpu.upload(np.asarray(t.data)), shape, t.dtype)
        self.consts[key] = val
        return val

    # ---- planning
    def _plan(self, s):
        if s in self.plans:
            return self.plans[s]
        g, pkg, nodes, uses = self.gpu, self.pkg, self.pkg.nodes, self.uses
        sym = {self.sym_seq: s, self.sym_ctx: self.capacity}
        plan = _Plan()
        vals, skip = {}, set()
        producer = {n.output: i for i, n in enumerate(nodes)}

        def new(shape, dtype):
            buf = g.alloc(max(_count(shape) * _ELEM[dtype], 4))
            plan.buffers.append(buf)
            return buf

        def emit(fn, *args, **kw):
            plan.steps.append((fn, args, kw))

        for vid, (idx, role) in self.roles.items():
            shape = pkg.shape_of(vid, sym)
            if role.kind == "sequence_cache":
                # retained_history_tokens > 0: a rolling ring (storage/aion_file/types.zig:195-197, storage/cache.zig:35-38)
                vals[vid] = _Val("dev", self.caches[idx], shape, "f16", extra="rolling" if role.retained_history_tokens else None)
                continue
            if role.kind not in ("tokens", "positions", "cache_write_index", "cache_visible_end"):
                raise Unsupported("input role %s" % role.kind)
            buf = new(shape, "i32")
            plan.inputs[role.kind] = (buf, shape)
            vals[vid] = _Val("dev", buf, shape, "i32")

        def get(vid):
            """The device value of `vid`; a pending cast is materialised."""
            if vid not in vals:
                if pkg.values[vid].source != "initializer":
                    raise PackageError("InvalidFormat", "value %d is read before it is produced" % vid)
                vals[vid] = self._const(vid)
            v = vals[vid]
            if v.kind == "cast":
                src = get(v.extra)
                out = new(v.shape, "f16")
                emit(g.step_cast_f32_f16, out, src.buf, _count(v.shape))
                v = vals[vid] = _Val("dev", out, v.shape, "f16")
            elif v.kind == "gelu":              # a gelu that does not feed a multiply: the plain unary step
                src = get(v.extra)
                out = new(v.shape, "f32")
                emit(g.step_unary, "gelu", out, src.buf, _count(v.shape))
                v = vals[vid] = _Val("dev", out, v.shape, "f32", owned=True)
            return v

        def weight_of(vid, allow_f32=False):
            """The matmul weight behind `vid`, or None. f32 weights (MatMulNT's plain operand) only where asked for: the
            fused steps are built on block dots."""
            if vid in vals:
                w = vals[vid]
            elif vid in producer and nodes[producer[vid]].op == "ViewTranspose2D":
                src = nodes[producer[vid]].inputs[0]
                if pkg.values[src].source != "initializer":
                    return None
                w = vals[vid] = self._const(src, transposed=True)
                skip.add(producer[vid])
            elif pkg.values[vid].source == "initializer":
                w = self._const(vid)
            else:
                return None
            return w if w.kind == "weight" and (allow_f32 or w.dtype != "f32") else None

        def sole_user(vid, op=None):
            """The one node that reads `vid` (None if it has several readers or is a graph output)."""
            u = uses.get(vid, [])
            if len(u) != 1 or u[0] == _OUT:
                return None
            return u[0] if op is None or nodes[u[0]].op in (op if isinstance(op, tuple) else (op,)) else None

        def residual_of(add_idx, produced_vid):
            """For add(res, produced) / add(produced, res): the value id of res if the sum may overwrite res."""
            n = nodes[add_idx]
            if n.op != "ElemwiseBinary" or n.attrs["op"] != "add" or produced_vid not in n.inputs or n.inputs[0] == n.inputs[1]:
                return None
            res = n.inputs[1] if n.inputs[0] == produced_vid else n.inputs[0]
            rv = vals.get(res)
            if rv is None or rv.kind != "dev" or not rv.owned or rv.dtype != "f32":
                return None
            if any(u > add_idx or (u != add_idx and nodes[u].op in _VIEWS + ("SequenceAppend",)) for u in uses.get(res, [])):
                return None
            if pkg.shape_of(res, sym) != pkg.shape_of(n.output, sym):
                return None
            return res

        def matmul_nodes_on(h_vid):
            """All readers of h are MatMuls with h on the left and a quantized weight on the right: their indices."""
            u = uses.get(h_vid, [])
            if not u or _OUT in u:
                return None
            out = []
            for i in u:
                n = nodes[i]
                if n.op != "MatMul" or n.inputs[0] != h_vid or n.attrs["beta"] != 0.0 or n.attrs["alpha"] != 1.0 or weight_of(n.inputs[1]) is None:
                    return None
                out.append(i)
            return out if len(set(weight_of(nodes[i].inputs[1]).dtype for i in out)) == 1 else None

        def try_qkv(i, mms):
            """One new token: RMSNorm -> q,k,v -> reshape -> RoPE1D(q,k) -> Cast -> SequenceAppend(k,v)."""
            if s != 1 or len(mms) != 3:
                return False
            n0 = nodes[i]
            x = get(n0.inputs[0])
            if x.shape[0] != 1 or x.shape[-1] > 8192:
                return False
            chains = {}
            for m in mms:
                r = sole_user(nodes[m].output, "ViewReshape")
                if r is None or len(pkg.shape_of(nodes[r].output, sym)) != 4:
                    return False
                nxt = sole_user(nodes[r].output)
                if nxt is None:
                    return False
                if nodes[nxt].op == "RoPE1D":
                    rope = nxt
                    after = sole_user(nodes[rope].output)
                    if after is None:
                        return False
                    if nodes[after].op == "Attention" and nodes[after].inputs[0] == nodes[rope].output:
                        chains["q"] = (m, r, rope)
                    elif nodes[after].op == "Cast":
                        app = sole_user(nodes[after].output, "SequenceAppend")
                        if app is None or nodes[app].inputs[1] != nodes[after].output:
                            return False
                        chains["k"] = (m, r, rope, after, app)
                    else:
                        return False
                elif nodes[nxt].op == "Cast":
                    app = sole_user(nodes[nxt].output, "SequenceAppend")
                    if app is None or nodes[app].inputs[1] != nodes[nxt].output:
                        return False
                    chains["v"] = (m, r, nxt, app)
                else:
                    return False
            if set(chains) != {"q", "k", "v"}:
                return False
            rq, rk = nodes[chains["q"][2]], nodes[chains["k"][2]]
            ak, av = nodes[chains["k"][4]], nodes[chains["v"][3]]
            if rq.attrs != rk.attrs or rq.inputs[1] != rk.inputs[1] or ak.inputs[2] != av.inputs[2]:
                return False
            if any(nodes[c].attrs["to_dtype"] != "f16" for c in (chains["k"][3], chains["v"][2])):
                return False
            qs, ks = pkg.shape_of(rq.output, sym), pkg.shape_of(rk.output, sym)
            if qs[:2] != (1, 1) or ks[:2] != (1, 1) or qs[3] != ks[3] or qs[3] % 8:
                return False
            kc, vc = get(ak.inputs[0]), get(av.inputs[0])
            if kc.shape != vc.shape or kc.shape[2:] != ks[2:] or kc.dtype != "f16" or kc.extra != vc.extra or kc.extra not in (None, "rolling"):
                return False
            gamma, beta = get(n0.inputs[1]), get(n0.inputs[2])
            q_out = new(qs, "f32")
            emit(g.step_rmsnorm_qkv_rope_append, weight_of(nodes[chains["q"][0]].inputs[1]).buf, weight_of(nodes[chains["k"][0]].inputs[1]).buf,
                 weight_of(nodes[chains["v"][0]].inputs[1]).buf, x.buf, gamma.buf, n0.attrs["eps"], q_out, kc.buf, vc.buf,
                 get(rq.inputs[1]).buf, get(ak.inputs[2]).buf, kc.shape[1], qs[2], ks[2], qs[3], base=rq.attrs["base_frequency"],
                 scale_factor=rq.attrs["scale_factor"], proportion=rq.attrs["rope_proportion"], beta_norm=beta.buf,
                 rolling=kc.extra == "rolling")
            vals[rq.output] = _Val("dev", q_out, qs, "f32", owned=True)
            vals[ak.output] = _Val("dev", kc.buf, kc.shape, "f16", extra=kc.extra)
            vals[av.output] = _Val("dev", vc.buf, vc.shape, "f16", extra=vc.extra)
            for c in chains.values():
                skip.update(c)
            return True

        def try_headnorm(i):
            """Per-head norms between the projections and the cache (src/bench/models.zig:455-473):
            q,k,v -> reshape -> RMSNorm over the head size -> RoPE1D(q,k) -> Cast -> SequenceAppend(k,v), one launch.
            Called at the first of the three norms; the three projections are already on the device."""
            n0 = nodes[i]
            r0 = producer.get(n0.inputs[0])
            if r0 is None or nodes[r0].op != "ViewReshape":
                return False
            m0 = producer.get(nodes[r0].inputs[0])
            if m0 is None or nodes[m0].op != "MatMul":
                return False
            sibs = uses.get(nodes[m0].inputs[0], [])
            if len(sibs) != 3 or _OUT in sibs or any(nodes[m].op != "MatMul" or nodes[m].output not in vals for m in sibs):
                return False
            chains, src = {}, {}
            for m in sibs:
                r = sole_user(nodes[m].output, "ViewReshape")
                if r is None or len(pkg.shape_of(nodes[r].output, sym)) != 4:
                    return False
                nrm = sole_user(nodes[r].output, "RMSNorm")
                if nrm is None or nodes[nrm].inputs[0] != nodes[r].output or nrm in skip or nrm < i:
                    return False
                hs = pkg.shape_of(nodes[nrm].output, sym)
                if [pkg.dim_term(t, sym) for t in nodes[nrm].attrs["normalized_shape"]] != [hs[3]]:
                    return False
                nxt = sole_user(nodes[nrm].output)
                if nxt is None:
                    return False
                if nodes[nxt].op == "RoPE1D" and nodes[nxt].inputs[0] == nodes[nrm].output:
                    after = sole_user(nodes[nxt].output)
                    if after is None:
                        return False
                    if nodes[after].op == "Attention" and nodes[after].inputs[0] == nodes[nxt].output:
                        chains["q"], src["q"] = (nrm, nxt), m
                    elif nodes[after].op == "Cast":
                        app = sole_user(nodes[after].output, "SequenceAppend")
                        if app is None or nodes[app].inputs[1] != nodes[after].output:
                            return False
                        chains["k"], src["k"] = (nrm, nxt, after, app), m
                    else:
                        return False
                elif nodes[nxt].op == "Cast":
                    app = sole_user(nodes[nxt].output, "SequenceAppend")
                    if app is None or nodes[app].inputs[1] != nodes[nxt].output:
                        return False
                    chains["v"], src["v"] = (nrm, nxt, app), m
                else:
                    return False
            if set(chains) != {"q", "k", "v"} or chains["q"][0] != i:
                return False
            nq, nk, nv = (nodes[chains[c][0]] for c in "qkv")
            rq, rk = nodes[chains["q"][1]], nodes[chains["k"][1]]
            ak, av = nodes[chains["k"][3]], nodes[chains["v"][2]]
            if rq.attrs != rk.attrs or rq.inputs[1] != rk.inputs[1] or ak.inputs[2] != av.inputs[2]:
                return False
            if nq.attrs["eps"] != nk.attrs["eps"] or nq.attrs["eps"] != nv.attrs["eps"]:
                return False
            if any(nodes[c].attrs["to_dtype"] != "f16" for c in (chains["k"][2], chains["v"][1])):
                return False
            qs, ks, vs = (pkg.shape_of(x.output, sym) for x in (nq, nk, nv))
            if qs[:2] != ks[:2] or ks != vs or qs[3] != ks[3] or qs[3] % 2 or qs[3] > 512:
                return False
            kc, vc = get(ak.inputs[0]), get(av.inputs[0])
            if kc.shape != vc.shape or kc.shape[0] != ks[0] or kc.shape[2:] != ks[2:] or kc.dtype != "f16" or kc.extra != vc.extra \
                    or kc.extra not in (None, "rolling") or ks[1] > kc.shape[1]:
                return False
            srcs = [get(nodes[src[c]].output) for c in "qkv"]          # the reshapes between are views of these
            if any(x.dtype != "f32" for x in srcs):
                return False
            gammas = [get(x.inputs[1]).buf for x in (nq, nk, nv)]
            betas = [get(x.inputs[2]).buf for x in (nq, nk, nv)]
            q_out = new(qs, "f32")
            emit(g.step_headnorm_rope_append, q_out, srcs[0].buf, srcs[1].buf, srcs[2].buf, gammas, betas, nq.attrs["eps"], kc.buf, vc.buf,
                 get(rq.inputs[1]).buf, get(ak.inputs[2]).buf, qs[0], qs[1], kc.shape[1], qs[2], ks[2], qs[3],
                 base=rq.attrs["base_frequency"], scale_factor=rq.attrs["scale_factor"], proportion=rq.attrs["rope_proportion"],
                 rolling=kc.extra == "rolling")
            vals[rq.output] = _Val("dev", q_out, qs, "f32", owned=True)
            vals[ak.output] = _Val("dev", kc.buf, kc.shape, "f16", extra=kc.extra)
            vals[av.output] = _Val("dev", vc.buf, vc.shape, "f16", extra=vc.extra)
            for c in chains.values():
                skip.update(c)
            return True

        def try_geglu(i, mms):
            """One new token: RMSNorm -> gate, up -> gelu(gate) * up -> down -> add(residual, .)."""
            if s != 1 or len(mms) != 2:
                return False
            n0 = nodes[i]
            x = get(n0.inputs[0])
            if _count(x.shape[:-1]) != 1 or x.shape[-1] > 8192:
                return False
            ge = [m for m in mms if sole_user(nodes[m].output, "Unary") is not None]
            if len(ge) != 1:
                return False
            mg = ge[0]
            mu = mms[0] if mms[1] == mg else mms[1]
            un = sole_user(nodes[mg].output, "Unary")
            if nodes[un].attrs["op"] != "gelu":
                return False
            mul = sole_user(nodes[un].output, "ElemwiseBinary")
            if mul is None or nodes[mul].attrs["op"] != "mul" or nodes[mul].inputs != (nodes[un].output, nodes[mu].output):
                return False
            if sole_user(nodes[mu].output) != mul:
                return False
            md = sole_user(nodes[mul].output, "MatMul")
            if md is None or nodes[md].inputs[0] != nodes[mul].output or nodes[md].attrs["beta"] != 0.0 or nodes[md].attrs["alpha"] != 1.0:
                return False
            wd = weight_of(nodes[md].inputs[1])
            if wd is None:
                return False
            add = sole_user(nodes[md].output, "ElemwiseBinary")
            res = residual_of(add, nodes[md].output) if add is not None else None
            wg, wu = weight_of(nodes[mg].inputs[1]), weight_of(nodes[mu].inputs[1])
            if wg.shape != wu.shape or wg.shape[1] % 32 or wd.dtype != wg.dtype:
                return False
            gamma, beta = get(n0.inputs[1]), get(n0.inputs[2])
            if res is not None:
                rv = vals[res]
                acc = rv.buf
                if self.keep_residuals:
                    acc = new(rv.shape, "f32")
                    emit(g.copy, acc, rv.buf, _count(rv.shape) * 4)
                emit(g.step_rmsnorm_geglu_matmul, wg.buf, wu.buf, wd.buf, x.buf, gamma.buf, n0.attrs["eps"], acc, beta=1.0, beta_norm=beta.buf)
                vals[nodes[add].output] = _Val("dev", acc, rv.shape, "f32", owned=True)
                skip.update((mg, mu, un, mul, md, add))
            else:                                   # the down projection feeds something else (a norm): a buffer of its own
                oshape = pkg.shape_of(nodes[md].output, sym)
                out = new(oshape, "f32")
                emit(g.step_rmsnorm_geglu_matmul, wg.buf, wu.buf, wd.buf, x.buf, gamma.buf, n0.attrs["eps"], out, beta=0.0, beta_norm=beta.buf)
                vals[nodes[md].output] = _Val("dev", out, oshape, "f32", owned=True)
                skip.update((mg, mu, un, mul, md))
            return True

        def matmul_into(out_vid, launch):
            """Emits `launch(c_buf, beta)` for a matmul-like step producing `out_vid`, folding a following residual add."""
            shape = pkg.shape_of(out_vid, sym)
            add = sole_user(out_vid, "ElemwiseBinary") if self.fuse else None
            res = residual_of(add, out_vid) if add is not None else None
            if res is not None:
                rv = vals[res]
                acc = rv.buf
                if self.keep_residuals:
                    acc = new(rv.shape, "f32")
                    emit(g.copy, acc, rv.buf, _count(rv.shape) * 4)
                launch(acc, 1.0)
                vals[nodes[add].output] = _Val("dev", acc, rv.shape, "f32", owned=True)
                skip.add(add)
            else:
                out = new(shape, "f32")
                launch(out, 0.0)
                vals[out_vid] = _Val("dev", out, shape, "f32", owned=True)

        for i, n in enumerate(nodes):
            if i in skip:
                continue
            shape = pkg.shape_of(n.output, sym)
            op, a = n.op, n.attrs
            if op == "Gather":
                table, ids = get(n.inputs[0]), get(n.inputs[1])
                if a["axis"] != 0 or a["batch_dims"] != 0 or len(table.shape) != 2 or table.dtype not in ("f32", "q8_0"):
                    raise Unsupported("Gather other than rows of an f32 or row-quantized q8_0 table")
                out = new(shape, "f32")
                emit(g.step_gather_rows, be.F32 if table.dtype == "f32" else be.Q8_0, out, table.buf, ids.buf, _count(ids.shape),
                     table.shape[1], table.shape[0])
                vals[n.output] = _Val("dev", out, shape, "f32", owned=True)
            elif op == "RMSNorm":
                x, gamma, beta = get(n.inputs[0]), get(n.inputs[1]), get(n.inputs[2])
                cols = 1
                for t in a["normalized_shape"]:
                    cols *= pkg.dim_term(t, sym)
                if cols != x.shape[-1]:
                    raise Unsupported("RMSNorm over more than the last axis")
                rows = _count(x.shape) // cols
                if self.fuse and len(x.shape) == 4 and try_headnorm(i):
                    continue
                mms = matmul_nodes_on(n.output) if self.fuse else None
                if mms and (try_qkv(i, mms) or try_geglu(i, mms)):
                    continue
                if mms and len(mms) <= 4:
                    ws = [weight_of(nodes[m].inputs[1]).buf for m in mms]
                    outs = [new(pkg.shape_of(nodes[m].output, sym), "f32") for m in mms]
                    emit(g.step_rmsnorm_matmul, ws, x.buf, gamma.buf, rows, outs, a["eps"], beta_norm=beta.buf)
                    for m, o in zip(mms, outs):
                        vals[nodes[m].output] = _Val("dev", o, pkg.shape_of(nodes[m].output, sym), "f32", owned=True)
                    skip.update(mms)
                    continue
                add = sole_user(n.output, "ElemwiseBinary") if self.fuse else None
                res = residual_of(add, n.output) if add is not None else None
                if res is not None and vals[res].buf is not x.buf:
                    # add(residual, norm(x)): the norm step's own residual operand, summed in place (the same two roundings)
                    rv = vals[res]
                    acc = new(rv.shape, "f32") if self.keep_residuals else rv.buf      # out-of-place needs no copy here
                    emit(g.step_rmsnorm, acc, x.buf, gamma.buf, rows, cols, a["eps"], beta=beta.buf, residual=rv.buf)
                    vals[nodes[add].output] = _Val("dev", acc, rv.shape, "f32", owned=True)
                    skip.add(add)
                    continue
                out = new(shape, "f32")
                emit(g.step_rmsnorm, out, x.buf, gamma.buf, rows, cols, a["eps"], beta=beta.buf)
                vals[n.output] = _Val("dev", out, shape, "f32", owned=True)
            elif op == "ViewTranspose2D":
                if weight_of(n.output, allow_f32=True) is None:
                    raise Unsupported("ViewTranspose2D of anything but a weight")
            elif op == "MatMul":
                x, w = get(n.inputs[0]), weight_of(n.inputs[1], allow_f32=True)
                if w is None:
                    raise Unsupported("MatMul whose right operand is not a weight")
                if a["beta"] != 0.0:
                    raise Unsupported("MatMul with beta != 0 in a package")
                m_rows, alpha = _count(x.shape[:-1]), a["alpha"]
                matmul_into(n.output, lambda c, beta, w=w, x=x, m_rows=m_rows, alpha=alpha:
                            emit(g.step_matmul, w.buf, x.buf, m_rows, c, alpha=alpha, beta=beta))
            elif op in _VIEWS:
                x = get(n.inputs[0])
                if _count(shape) != _count(x.shape):
                    raise PackageError("InvalidFormat", "view changes the element count")
                vals[n.output] = _Val("dev", x.buf, shape, x.dtype)
            elif op == "RoPE1D":
                x, pos = get(n.inputs[0]), get(n.inputs[1])
                if len(x.shape) != 4:
                    raise Unsupported("RoPE1D on rank %d" % len(x.shape))
                out = new(shape, "f32")
                emit(g.step_rope, out, x.buf, pos.buf, x.shape[0], x.shape[1], x.shape[2], x.shape[3], base=a["base_frequency"],
                     scale_factor=a["scale_factor"], proportion=a["rope_proportion"])
                vals[n.output] = _Val("dev", out, shape, "f32", owned=True)
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
                emit(g.step_append_f16, cache.buf, src.buf, widx.buf, cache.shape[0], newv.shape[1], cache.shape[1], _count(cache.shape[2:]),
                     rolling=cache.extra == "rolling")
                vals[n.output] = _Val("dev", cache.buf, shape, "f16", extra=cache.extra)
            elif op == "Attention":
                q, k, v = get(n.inputs[0]), get(n.inputs[1]), get(n.inputs[2])
                rest = list(n.inputs[3:])
                pos = get(rest.pop(0)) if a["has_query_positions"] else None
                lens = get(rest.pop(0)) if a["has_kv_lengths"] else None
                w = a["window"]
                out = new(shape, "f32")
                dts = {"f32": be.F32, "f16": be.F16}
                emit(g.step_attention, out, q.buf, k.buf, v.buf,
                     (q.shape[0], q.shape[1], k.shape[1], q.shape[2], k.shape[2], q.shape[3], v.shape[3]), a["scale"],
                     q_dtype=dts[q.dtype], kv_dtype=dts[k.dtype], window=(w["left"], w["right"], w["chunk"]), soft_cap=a["soft_cap"],
                     query_positions=pos.buf if pos else None, kv_lengths=lens.buf if lens else None,
                     rolling=k.extra == "rolling")
                vals[n.output] = _Val("dev", out, shape, "f32", owned=True)
            elif op == "Unary":
                if a["op"] == "gelu":           # pending: gelu(gate) * up is aion's gate step
                    vals[n.output] = _Val("gelu", None, shape, "f32", extra=n.inputs[0])
                elif a["op"] in ("relu", "silu", "sigmoid", "tanh", "sqrt"):
                    x = get(n.inputs[0])
                    out = new(shape, "f32")
                    emit(g.step_unary, a["op"], out, x.buf, _count(shape))
                    vals[n.output] = _Val("dev", out, shape, "f32", owned=True)
                else:
                    raise Unsupported("Unary %s" % a["op"])
            elif op == "ElemwiseBinary":
                lhs = vals.get(n.inputs[0])
                if a["op"] in ("add", "sub", "mul", "div") and not (a["op"] == "mul" and lhs is not None and lhs.kind == "gelu"):
                    # same shape, a scalar, or a contiguous suffix of the left operand's shape (cpu/exec/elementwise.zig:38-60)
                    x, y = get(n.inputs[0]), get(n.inputs[1])
                    if x.dtype != "f32" or y.dtype != "f32":
                        raise Unsupported("ElemwiseBinary on %s" % x.dtype)
                    ys = tuple(d for d in y.shape)
                    while len(ys) > 1 and ys[0] == 1:
                        ys = ys[1:]
                    if not (x.shape == y.shape or _count(ys) == 1 or (len(ys) <= len(x.shape) and tuple(x.shape[len(x.shape) - len(ys):]) == ys)):
                        raise Unsupported("ElemwiseBinary with a general broadcast")
                    if tuple(shape) != tuple(x.shape):
                        raise Unsupported("ElemwiseBinary that broadcasts its left operand")
                    out = new(shape, "f32")
                    if a["op"] == "add" and x.shape == y.shape:
                        emit(g.step_add, out, x.buf, y.buf, _count(shape))
                    else:
                        emit(g.step_binary, a["op"], out, x.buf, y.buf, _count(shape), _count(ys))
                    vals[n.output] = _Val("dev", out, shape, "f32", owned=True)
                elif a["op"] == "mul":
                    gate, up = get(lhs.extra), get(n.inputs[1])
                    md = sole_user(n.output, "MatMul") if self.fuse else None
                    wd = weight_of(nodes[md].inputs[1]) if md is not None and nodes[md].inputs[0] == n.output else None
                    if wd is not None and nodes[md].attrs["beta"] == 0.0:
                        rows, alpha = _count(gate.shape[:-1]), nodes[md].attrs["alpha"]
                        matmul_into(nodes[md].output, lambda c, beta, wd=wd, gate=gate, up=up, rows=rows, alpha=alpha:
                                    emit(g.step_gate_matmul, wd.buf, gate.buf, up.buf, rows, c, alpha=alpha, beta=beta))
                        skip.add(md)
                    else:
                        out = new(shape, "f32")
                        emit(g.step_gate_gelu, out, gate.buf, up.buf, _count(shape))
                        vals[n.output] = _Val("dev", out, shape, "f32", owned=True)
                else:
                    raise Unsupported("ElemwiseBinary %s" % a["op"])
            elif op == "ArgMax":
                x = get(n.inputs[0])
                if a["axis"] not in (-1, len(x.shape) - 1):
                    raise Unsupported("ArgMax over an inner axis")
                out = new(shape, "i32")
                emit(g.step_argmax, out, x.buf, _count(x.shape[:-1]), x.shape[-1])
                vals[n.output] = _Val("dev", out, shape, "i32", owned=True)
            else:
                raise Unsupported("operation %s has no step on this backend" % op)
        for name, vid in pkg.outputs:
            v = get(vid)
            plan.outputs[name] = (v.buf, v.shape, v.dtype)
        # every value that ended up in a device buffer of its own, by value id (fused-away values are absent): lets a
        # caller read an intermediate result after a run
        plan.values = {vid: (v.buf, v.shape, v.dtype) for vid, v in vals.items() if v.kind == "dev" and v.buf is not None}
        self.plans[s] = plan
        return plan

    # ---- running
    def _write_inputs(self, plan, tokens, pos):
        s = len(tokens)
        feeds = {"tokens": tokens, "positions": np.arange(pos, pos + s, dtype=np.int32),
                 "cache_write_index": np.array([pos], np.int32), "cache_visible_end": np.array([pos + s], np.int32)}
        for kind, (buf, shape) in plan.inputs.items():
            if _count(shape) != feeds[kind].size:
                raise PackageError("InvalidArgument", "input %s: shape %s for %d elements" % (kind, shape, feeds[kind].size))
            self.gpu.write(buf, feeds[kind])

    def _issue(self, plan):
        for fn, args, kw in plan.steps:
            fn(*args, **kw)

    def _read(self, plan, want):
        np_t = {"f32": np.float32, "i32": np.int32, "f16": np.float16}
        return {name: self.gpu.download(buf, np_t[dt], shape) for name, (buf, shape, dt) in plan.outputs.items() if name in want}

    # ---- cache growth
    def _required(self, s, pos=None):
        """Rows the caches must hold for a run of s tokens at position pos (self.pos if not given;
        api/loaded_model/sequence_cache.zig:45-51)."""
        pos = self.pos if pos is None else pos
        need = 0
        for idx, (_vid, retained, fixed_rows) in self.cache_meta.items():
            rows = (min(pos, retained) if retained else pos) + s
            if fixed_rows is None:
                need = max(need, rows)
            elif rows > fixed_rows:             # a cache of constant shape (a local layer's ring): nothing to grow
                raise ValueError("the run needs %d rows of cache input %d, which holds %d" % (rows, idx, fixed_rows))
        return need

    def _grow(self, required):
        g, gr = self.gpu, self.growth
        num, den = (2, 1) if self.all_rolling else (int(gr["numerator"]), int(gr["denominator"]))
        ceiling = 0 if self.all_rolling else int(gr.get("max_capacity", 0))
        target = self.capacity
        while target < required:
            target = g.cache_grow_target(target, num, den)
        p2 = 1
        while p2 < target:
            p2 *= 2
        target = max(p2, self.capacity * 4)
        if ceiling:
            if required > ceiling:
                raise ValueError("the run exceeds the caches' growth ceiling")
            target = min(target, ceiling)
        ends = None
        for idx, (vid, retained, fixed_rows) in self.cache_meta.items():
            if fixed_rows is not None:
                continue
            old_shape = self.pkg.shape_of(vid, {self.sym_ctx: self.capacity, self.sym_seq: 1})
            new_shape = self.pkg.shape_of(vid, {self.sym_ctx: target, self.sym_seq: 1})
            if old_shape[1] != self.capacity or new_shape[1] != target or old_shape[:1] + old_shape[2:] != new_shape[:1] + new_shape[2:]:
                raise Unsupported("cache input %d: the capacity symbol is not its time axis" % idx)
            b, row_bytes = old_shape[0], _count(old_shape[2:]) * 2
            new = g.alloc(_count(new_shape) * 2)          # every byte is written by the growth kernel
            if retained:
                if ends is None:
                    ends = g.upload(np.full(b, self.pos, np.int32))
                g.cache_grow_rolling(new, self.caches[idx], ends, b, self.capacity, target, row_bytes, retained)
            else:
                g.cache_grow(new, self.caches[idx], b, self.capacity * row_bytes, target * row_bytes)
            g.sync()
            self.caches[idx].free()
            self.caches[idx] = new
        if ends is not None:
            ends.free()
        # every plan holds the old caches and the old capacity in its shapes
        if self.program is not None:
            g.program_destroy(self.program)
            self.program = None
        for plan in self.plans.values():
            for buf in plan.buffers:
                buf.free()
        self.plans = {}
        self.capacity = target

    def _ensure_capacity(self, s):
        required = self._required(s)
        if required <= self.capacity:
            return
        if self.growth is None:
            raise ValueError("the run exceeds the cache capacity")
        self._grow(required)

    def run(self, tokens, want=("next_token",)):
        """Feeds `tokens` (int32 [S]) at positions pos..pos+S-1, runs the graph, advances pos. Returns the
        requested outputs (by signature name) as numpy arrays."""
        tokens = np.ascontiguousarray(tokens, np.int32).reshape(-1)
        self._ensure_capacity(tokens.size)
        plan = self._plan(tokens.size)
        self._write_inputs(plan, tokens, self.pos)
        self._issue(plan)
        out = self._read(plan, want)
        self.pos += tokens.size
        return out

    def step_count(self, s=1):
        return len(self._plan(s).steps)

    def begin_decode(self, first_token, token_output="next_token"):
        """Records the one-token plan as a program whose loop state stays on the device: the token the graph
        produced becomes the next run's token, position / write index / visible end advance by one."""
        g = self.gpu
        plan = self._plan(1)
        self._write_inputs(plan, np.array([first_token], np.int32), self.pos)
        if self.program is not None and not g.program_is_current(self.program):
            # a larger run since the recording made the context replace a work buffer the program's launches address
            g.program_destroy(self.program)
            self.program = None
        if self.program is None:
            self._issue(plan)                    # eager once: scratch buffers reach their final size
            g.sync()
            self._write_inputs(plan, np.array([first_token], np.int32), self.pos)
            if self.one is None:
                self.one = g.upload(np.ones(1, np.int32))
            tok_buf = plan.outputs[token_output][0]

            if self.log is None:
                # the tokens a run of replays produces, logged on the device at a counter of their own (decode_run reads them
                # once per run; the counter is one more value the state-advance launch moves)
                self.log = g.alloc(self.LOG_TOKENS * 4)
                self.log_at = g.upload(np.zeros(1, np.int32))

            def issue():
                self._issue(plan)
                g.step_advance_state(plan.inputs["tokens"][0], tok_buf, 1,
                                     [plan.inputs[kind][0] for kind in ("positions", "cache_write_index", "cache_visible_end")] + [self.log_at],
                                     log=self.log, log_index=self.log_at, log_capacity=self.LOG_TOKENS)
            self.program = g.record_program(issue)
        self._token_output = token_output

    def decode_step(self, read_token=True):
        if self._required(1) > self.capacity:
            if self.growth is None:
                raise ValueError("cache capacity exhausted")
            # the loop state lives in the old plan's buffers: take the pending token out, grow, record again
            token = int(self.gpu.download(self.plans[1].inputs["tokens"][0], np.int32, (1,))[0])
            self._grow(self._required(1))
            self.begin_decode(token, self._token_output)
        self.gpu.program_execute(self.program)
        self.pos += 1
        if read_token:
            buf, shape, _ = self.plans[1].outputs[self._token_output]
            return int(self.gpu.download(buf, np.int32, shape).reshape(-1)[-1])
        return None

    def decode_run(self, n):
        """n replays of the decode program with nothing read back in between: the produced tokens are logged on the device
        and collected once per stretch of replays (a stretch ends where the caches have to grow, or the log is full)."""
        out = []
        while n > 0:
            if self._required(1) > self.capacity:
                if self.growth is None:
                    raise ValueError("cache capacity exhausted")
                token = int(self.gpu.download(self.plans[1].inputs["tokens"][0], np.int32, (1,))[0])
                self._grow(self._required(1))
                self.begin_decode(token, self._token_output)
            c = 1                                # single-token runs that fit the caches as they are
            while c < min(n, self.LOG_TOKENS) and self._required(1, self.pos + c) <= self.capacity:
                c += 1
            self.gpu.write(self.log_at, np.zeros(1, np.int32))
            for _ in range(c):
                self.gpu.program_execute(self.program)
            self.pos += c
            out.extend(int(t) for t in self.gpu.download(self.log, np.int32, (c,)))
            n -= c
        return out

    def reset(self):
        self.pos = 0

    def close(self):
        if self.program is not None:
            self.gpu.program_destroy(self.program)
            self.program = None
        for plan in self.plans.values():
            for b in plan.buffers:
                b.free()
        for c in self.consts.values():
            c.buf.free()
        for b in self.caches.values():
            b.free()
        if self.one is not None:
            self.one.free()
        if self.log is not None:
            self.log.free(); self.log_at.free()
        self.plans, self.consts, self.caches, self.one, self.log, self.log_at = {}, {}, {}, None, None, None
