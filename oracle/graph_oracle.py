"""Test infrastructure, not product code: a node-by-node CPU interpreter for decoder graphs held in `.aion` packages,
built from the oracle's restatements of aion's CPU steps (oracle/oracle.py). It is the checker for what
aion_amd/package.py schedules on the GPU: every node is evaluated on its own, in file order, with no fusion, which
is what aion's CPU backend computes for the same graph before its step fusions (those are bit-preserving:
cpu/exec/elementwise.zig:25-37). Pinned by tests/test_graph_oracle.py against the hand-written C++ oracle decoder
on the plain decoder package (same weights, same tokens -> the same logits).

Takes a parsed package (any object with the fields of aion_amd.aion_file.Package) so that the oracle does not carry a
second reader; the reader itself is pinned by round trips against oracle/aion_writer.py."""
import numpy as np

from . import oracle as orc

_NP = {"f32": np.float32, "f16": np.float16, "i32": np.int32}
_VIEWS = ("ViewReshape", "ViewSqueeze", "ViewUnsqueeze")


class _Quant:
    """A block-quantized initializer: logical shape, scheme, packed blocks; `transposed` after a ViewTranspose2D."""

    def __init__(self, scheme, quant_axis, shape, blocks, transposed=False):
        self.scheme, self.quant_axis, self.shape, self.blocks, self.transposed = scheme, quant_axis, tuple(shape), blocks, transposed


class _PlainT:
    """The ViewTranspose2D of a plain f32 [N,K] initializer: the right operand of a MatMulNT with an f32 B."""

    def __init__(self, rows):
        self.rows = rows


def _initializer(pkg, vid):
    v = pkg.values[vid]
    t = pkg.tensors[v.initializer]
    shape = pkg.shape_of(vid, {})
    if t.quantized:
        return _Quant(t.scheme, t.quant_axis, shape, np.asarray(t.data))
    return np.asarray(t.data).view(_NP[t.dtype]).reshape(shape)        # a read-only view of the payload, no copy


def _matmul(x, w, alpha, attn_threads):
    m = int(np.prod(x.shape[:-1]))
    a = x.reshape(m, x.shape[-1])
    if isinstance(w, _PlainT):                                                 # graph/program/compiler.zig:337-357: MatMulNT, f32 B
        return orc.matmul_nt_f32(a, w.rows, alpha=alpha)
    if w.scheme == "q4_0" and w.quant_axis == 0 and not w.transposed:          # [K,N] packed along K
        return orc.matmul_q_packed(orc.Q4_0, a, w.blocks, w.shape[1], alpha=alpha, threads=attn_threads)
    if w.scheme == "q8_0" and w.quant_axis == 0 and not w.transposed:
        return orc.matmul_q_packed(orc.Q8_0, a, w.blocks, w.shape[1], alpha=alpha, threads=attn_threads)
    if w.scheme == "q8_0" and w.quant_axis == 1 and w.transposed:              # [N,K] rows, used as its transpose
        return orc.matmul_nt_q8(a, w.blocks, w.shape[0], alpha=alpha, threads=attn_threads)
    raise ValueError("graph oracle: no matmul for %s quant_axis %d%s" % (w.scheme, w.quant_axis, " transposed" if w.transposed else ""))


def _eval(pkg, n, ins, a, ring, exact_attention, round_q_f16, threads):
    """One node on the given input values. Returns the output (unshaped), or a _Quant for a weight view."""
    if n.op == "Gather":
        table, ids = ins
        if a["axis"] != 0 or a["batch_dims"] != 0:
            raise ValueError("graph oracle: Gather axis 0 only")
        if isinstance(table, _Quant):
            if table.scheme != "q8_0" or table.quant_axis != 1:
                raise ValueError("graph oracle: a quantized gather table is q8_0 along its rows")
            return orc.gather_rows(table.blocks, ids.reshape(-1), table.shape[1], dtype=1)
        return orc.gather_rows(table, ids.reshape(-1), table.shape[1])
    if n.op == "RMSNorm":
        x, gamma, beta = ins
        return orc.rmsnorm(x.reshape(-1, x.shape[-1]), gamma, a["eps"], beta=beta)
    if n.op == "ViewTranspose2D":
        w = ins[0]
        if isinstance(w, np.ndarray) and w.dtype == np.float32 and w.ndim == 2:
            return _PlainT(w)
        if not isinstance(w, _Quant):
            raise ValueError("graph oracle: ViewTranspose2D of a weight only")
        return _Quant(w.scheme, w.quant_axis, w.shape, w.blocks, transposed=not w.transposed)
    if n.op == "MatMul":
        if a["beta"] != 0.0:
            raise ValueError("graph oracle: MatMul beta")
        return _matmul(ins[0], ins[1], a["alpha"], threads)
    if n.op in _VIEWS:
        return ins[0]
    if n.op == "RoPE1D":
        return orc.rope(ins[0], ins[1], base=a["base_frequency"], scale_factor=a["scale_factor"], proportion=a["rope_proportion"])
    if n.op == "Cast":
        if a["to_dtype"] != "f16":
            raise ValueError("graph oracle: Cast to f16 only")
        return orc.cast_f32_f16(ins[0])
    if n.op == "SequenceAppend":
        cache, new, end = ins
        return orc.sequence_append(cache, new.reshape((cache.shape[0], -1) + cache.shape[2:]), end.reshape(-1), rolling=ring)
    if n.op == "Attention":
        q, k, v = ins[:3]
        if round_q_f16:
            q = q.astype(np.float16).astype(np.float32)
        rest = list(ins[3:])
        pos = rest.pop(0) if a["has_query_positions"] else None
        lens = rest.pop(0) if a["has_kv_lengths"] else None
        w = a["window"]
        window = (w["left"], w["right"], w["chunk"])
        if ring:
            return orc.attention_rolling_f64(q, k.astype(np.float32), v.astype(np.float32), a["scale"], window,
                                             pos.reshape(q.shape[0], -1), lens.reshape(-1), soft_cap=a["soft_cap"])
        fn = orc.attention_f64 if exact_attention else orc.attention_blocked
        return fn(q, k, v, a["scale"], window=window, soft_cap=a["soft_cap"],
                  positions=None if pos is None else pos.reshape(q.shape[0], -1), kv_lengths=None if lens is None else lens.reshape(-1))
    if n.op == "Unary":
        return orc.unary(a["op"], ins[0])
    if n.op == "ElemwiseBinary":
        return orc.binary(a["op"], ins[0], ins[1])
    if n.op == "ArgMax":
        return orc.argmax(ins[0].reshape(-1, ins[0].shape[-1]))
    raise ValueError("graph oracle: no restatement for %s" % n.op)


def _start(pkg, feeds, rolling_inputs):
    vals, rolling = {}, set()
    for name, vid in pkg.inputs:
        vals[vid] = np.asarray(feeds[name])
        if name in rolling_inputs:
            rolling.add(vid)
    # initializers are immutable: materialised once per package object (a 2-billion-parameter package is evaluated many times)
    inits = getattr(pkg, "_graph_oracle_initializers", None)
    if inits is None:
        inits = {vid: _initializer(pkg, vid) for vid, v in enumerate(pkg.values) if v.initializer is not None}
        try:
            pkg._graph_oracle_initializers = inits
        except AttributeError:
            pass
    vals.update(inits)
    return vals, rolling


def run_graph(pkg, feeds, symbols, rolling_inputs=(), exact_attention=False, round_q_f16=False, threads=4):
    """Evaluates every node. feeds: input name -> array (caches included, f16); symbols: dimension symbol -> value;
    rolling_inputs: names of cache inputs that are rings. Returns {output name: array}.
    round_q_f16: the queries of every Attention are rounded to f16 first - a second evaluation that differs from the
    first by one operand rounding (the one the GPU's MFMA kernels apply), which measures how much of a difference
    the graph itself amplifies (int8 activation codes flip under the smallest perturbation)."""
    vals, rolling = _start(pkg, feeds, rolling_inputs)
    for n in pkg.nodes:
        ring = n.op in ("SequenceAppend", "Attention") and n.inputs[0 if n.op == "SequenceAppend" else 1] in rolling
        out = _eval(pkg, n, [vals[i] for i in n.inputs], n.attrs, ring, exact_attention, round_q_f16, threads)
        if n.op == "SequenceAppend" and ring:
            rolling.add(n.output)
        vals[n.output] = out if isinstance(out, (_Quant, _PlainT)) else np.asarray(out).reshape(pkg.shape_of(n.output, symbols))
    return {name: vals[vid] for name, vid in pkg.outputs}


def check_nodes(pkg, feeds, symbols, device_values, rolling_inputs=(), threads=4, sample_rows_over=None, with_carried=False):
    """Every node on its own: evaluated here on the inputs THE DEVICE produced (device_values: value id -> array, read
    back after a node-by-node run) and compared with the device's output of that node. Unlike an end-to-end comparison
    this does not let one node's rounding be amplified by the next ones. A SequenceAppend is skipped (its cache operand
    is updated in place, the earlier contents are gone) and so is a node with an operand the device did not keep.
    sample_rows_over: a MatMul whose output has more elements than this is evaluated on its first, middle and last
    activation row only (rows never interact), and those rows are compared.
    Returns [(node index, op, max|device - here| / rms(here))]; with_carried adds a fourth field: True when an operand
    was not the device's but carried on this side from the last values the device did keep (a fused schedule folds
    values into its neighbours: the node then checks the whole folded chain, roundings of the chain included)."""
    vals, rolling = _start(pkg, feeds, rolling_inputs)
    vals.update({vid: np.asarray(v) for vid, v in device_values.items()})
    carried = set()
    report = []
    for i, n in enumerate(pkg.nodes):
        if n.op == "SequenceAppend":
            if n.inputs[0] in rolling:
                rolling.add(n.output)
            continue
        if any(v not in vals for v in n.inputs):
            continue
        ring = n.op == "Attention" and n.inputs[1] in rolling
        ins = [vals[v] for v in n.inputs]
        from_carried = any(v in carried for v in n.inputs)
        rows = None
        if (sample_rows_over is not None and n.op == "MatMul" and n.output in device_values and not isinstance(ins[0], _Quant)
                and int(np.prod(pkg.shape_of(n.output, symbols))) > sample_rows_over):
            m = int(np.prod(ins[0].shape[:-1]))
            rows = sorted({0, m // 2, m - 1})
            ins = [ins[0].reshape(m, ins[0].shape[-1])[rows]] + ins[1:]
        out = _eval(pkg, n, ins, n.attrs, ring, False, False, threads)
        if isinstance(out, (_Quant, _PlainT)):
            vals[n.output] = out
            continue
        if rows is not None:
            ref = np.asarray(out).astype(np.float64).reshape(len(rows), -1)
            dev = np.asarray(device_values[n.output]).astype(np.float64).reshape(m, -1)[rows]
            rms = float(np.sqrt((ref ** 2).mean())) + 1e-30
            report.append((i, n.op, float(np.abs(dev - ref).max()) / rms) + ((from_carried,) if with_carried else ()))
            continue
        out = np.asarray(out).reshape(pkg.shape_of(n.output, symbols))
        if n.output in device_values:
            ref = out.astype(np.float64)
            rms = float(np.sqrt((ref ** 2).mean())) + 1e-30
            report.append((i, n.op, float(np.abs(np.asarray(device_values[n.output]).astype(np.float64) - ref).max()) / rms)
                          + ((from_carried,) if with_carried else ()))
        else:
            vals[n.output] = out          # a view or a value the device folded into a neighbour: carry this side's
            if n.op not in _VIEWS or from_carried:
                carried.add(n.output)
    return report
