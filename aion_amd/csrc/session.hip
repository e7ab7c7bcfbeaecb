// A session over a step list: the native twin of aion's Session.execute(prog) (backend/backend.zig:24-52) for the steps of
// a quantized decoder. Host code only: every step ends in one of the library's own aionhip_step_* entry points, so a list
// run here gives what the separate calls give.
//
// The list is checked as a whole before its first launch (tags, dtypes, shapes), the way the reference validates a program
// before it executes it (runtime/executable.zig:413-470 validate): a list with a step this device does not run fails with
// nothing done.
#include "common.h"

#include <cmath>
#include <cstring>
#include <initializer_list>
#include <map>
#include <utility>
#include <tuple>
#include <vector>

namespace {

struct Range {
    uint64_t lo = 0, hi = 0;
    bool overlaps(const Range &o) const { return lo < o.hi && o.lo < hi; }
};

size_t elems(const aionhip_tensor_ref &t) {
    size_t n = 1;
    for (uint32_t d = 0; d < t.rank; ++d) n *= (size_t)t.shape[d];
    return n;
}
// bytes of a tensor as aion stores it: 34 / 18 bytes per 32 elements for the block formats (backend/types.zig:41-59)
size_t bytes_of(const aionhip_tensor_ref &t) {
    const size_t n = elems(t);
    switch (t.dtype) {
    case AIONHIP_F32: case AIONHIP_I32: return n * 4;
    case AIONHIP_F16: case AIONHIP_BF16: return n * 2;
    case AIONHIP_I8: return n;
    case AIONHIP_Q8_0: return n / 32 * 34;
    case AIONHIP_Q4_0: return n / 32 * 18;
    default: return 0;
    }
}
Range range_of(const aionhip_tensor_ref &t) { return Range{t.handle, t.handle + bytes_of(t)}; }
size_t rows_of(const aionhip_tensor_ref &t) {
    size_t r = 1;
    for (uint32_t d = 0; d + 1 < t.rank; ++d) r *= (size_t)t.shape[d];
    return r;
}

// operands a step reads and writes, as address ranges (workspace slots are reused, so tensors are told apart by range)
struct Access {
    Range reads[7];
    int n_reads = 0;
    Range writes[1];
    int n_writes = 0;
};
Access access_of(const aionhip_step &st) {
    Access a;
    for (int i = 0; i < 5; ++i)
        if (st.in[i].handle) a.reads[a.n_reads++] = range_of(st.in[i]);
    const bool is_matmul = st.tag == AIONHIP_STEP_MATMUL || st.tag == AIONHIP_STEP_MATMUL_NT;
    if (st.tag == AIONHIP_STEP_TRANSFER && st.to_host) return a;
    if (st.out.handle) {
        a.writes[a.n_writes++] = range_of(st.out);
        // C of a matmul with beta != 0 and the cache of an append are read as well
        if ((is_matmul && st.beta != 0.f) || st.tag == AIONHIP_STEP_SEQUENCE_APPEND) a.reads[a.n_reads++] = range_of(st.out);
    }
    return a;
}
bool reads_range(const aionhip_step &st, const Range &r) {
    const Access a = access_of(st);
    for (int i = 0; i < a.n_reads; ++i)
        if (a.reads[i].overlaps(r)) return true;
    return false;
}
bool writes_range(const aionhip_step &st, const Range &r) {
    const Access a = access_of(st);
    for (int i = 0; i < a.n_writes; ++i)
        if (a.writes[i].overlaps(r)) return true;
    return false;
}
bool same_tensor(const aionhip_tensor_ref &a, const aionhip_tensor_ref &b) {
    return a.handle == b.handle && a.dtype == b.dtype && elems(a) == elems(b);
}

}  // namespace

struct aionhip_session {
    aionhip_ctx *ctx = nullptr;
    int fusion = AIONHIP_FUSE_SIBLINGS | AIONHIP_FUSE_WORKSPACE;
    // re-laid weights by (address, dtype, layout, n, k): built at first use from the blocks on the device
    std::map<std::tuple<uint64_t, int, int, size_t, size_t>, aionhip_weight *> weights;
    uint64_t calls_last_execute = 0;

    int fail(size_t index, const aionhip_step &st, int status, const char *why) {
        return set_err(ctx, status, "session step %zu (tag %d): %s", index, st.tag, why);
    }
    // a failing entry point has left its own message: keep it and put the step in front
    int wrap(size_t index, const aionhip_step &st, int rc) {
        if (rc == AIONHIP_OK) return rc;
        char inner[384];
        snprintf(inner, sizeof inner, "%s", aionhip_last_error(ctx));
        return set_err(ctx, rc, "session step %zu (tag %d): %s", index, st.tag, inner);
    }

    void drop_weights() {
        for (auto &kv : weights) aionhip_weight_free(ctx, kv.second);
        weights.clear();
    }

    int weight_for(const aionhip_tensor_ref &b, int layout, aionhip_weight **out) {
        const size_t n = layout == AIONHIP_ROWS_NK ? b.shape[0] : b.shape[1];
        const size_t k = layout == AIONHIP_ROWS_NK ? b.shape[1] : b.shape[0];
        const auto key = std::make_tuple((uint64_t)b.handle, (int)b.dtype, layout, n, k);
        auto it = weights.find(key);
        if (it != weights.end()) { *out = it->second; return AIONHIP_OK; }
        if (ctx->capturing) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "a weight's first use falls inside a recording: run the list once eagerly first");
        aionhip_weight *w = nullptr;
        const int rc = aionhip_weight_from_device(ctx, b.dtype, layout, n, k, 0, b.handle, &w);
        if (rc) return rc;
        weights.emplace(key, w);
        *out = w;
        return AIONHIP_OK;
    }

    int check(size_t i, const aionhip_step &st);
    int check_list(const aionhip_step *steps, size_t count);
    int run_one(size_t i, const aionhip_step &st);
    // the value a pattern ending at step `last` would leave unwritten in `t`: true when no step behind `last` reads it before it
    // is overwritten in full (and - the tensor being a workspace tensor - nothing reads it after the list)
    bool only_read_within(const aionhip_step *steps, size_t count, size_t last, const aionhip_tensor_ref &t) const;
    size_t try_fused(const aionhip_step *steps, size_t count, size_t i, int *rc);
    // steps[j]: a MatMul with beta 0 into a workspace tensor T that only the step right behind it reads, that step being an
    // add that accumulates in place (X = X + T or X = T + X). The matmul may then write X itself with beta 1: alpha * acc + X
    // is rounded once either way. Returns X's address, or 0 when the two steps are not of that form.
    aionhip_handle residual_target(const aionhip_step *steps, size_t count, size_t j) const;
};

namespace {

bool is_f32(const aionhip_tensor_ref &t) { return t.handle && t.dtype == AIONHIP_F32; }
bool is_i32(const aionhip_tensor_ref &t) { return t.handle && t.dtype == AIONHIP_I32; }
bool is_matmul_tag(int tag) { return tag == AIONHIP_STEP_MATMUL || tag == AIONHIP_STEP_MATMUL_NT; }

// The cache side of an attention block among consecutive steps: RoPE1D on q and k, Cast f16 + SequenceAppend of k and of v,
// with or without an RMSNorm over the head size in front of each of q, k and v - in whatever order a valid program has them.
struct KvTail {
    const aionhip_step *norm[3] = {nullptr, nullptr, nullptr};      // sorted: q's, k's, v's
    const aionhip_step *rope[2] = {nullptr, nullptr};               // q's, k's
    const aionhip_step *cast[2] = {nullptr, nullptr};               // k's, v's
    const aionhip_step *app[2] = {nullptr, nullptr};                // k's, v's
};
// steps [lo, hi) are exactly `norms` head norms (0 or 3), two ropes, two casts and two appends wired as above
bool sort_kv_tail(const aionhip_step *steps, size_t lo, size_t hi, int norms, KvTail &t) {
    int n_norm = 0, n_rope = 0, n_cast = 0, n_app = 0;
    const aionhip_step *norm[3] = {nullptr, nullptr, nullptr};
    for (size_t j = lo; j < hi; ++j) {
        const aionhip_step &w = steps[j];
        if (w.tag == AIONHIP_STEP_RMSNORM && n_norm < norms && !w.in[3].handle) norm[n_norm++] = &w;
        else if (w.tag == AIONHIP_STEP_ROPE1D && n_rope < 2) t.rope[n_rope++] = &w;
        else if (w.tag == AIONHIP_STEP_CAST && n_cast < 2) t.cast[n_cast++] = &w;
        else if (w.tag == AIONHIP_STEP_SEQUENCE_APPEND && n_app < 2) t.app[n_app++] = &w;
        else return false;
    }
    if (n_norm != norms || n_rope != 2 || n_cast != 2 || n_app != 2) return false;
    // the cast that reads a rope's output is k's; that rope is k's, the other one q's, whose output leaves the pattern
    if (!same_tensor(t.cast[0]->in[0], t.rope[0]->out) && !same_tensor(t.cast[0]->in[0], t.rope[1]->out)) std::swap(t.cast[0], t.cast[1]);
    if (!same_tensor(t.cast[0]->in[0], t.rope[1]->out)) std::swap(t.rope[0], t.rope[1]);
    if (!same_tensor(t.app[0]->in[0], t.cast[0]->out)) std::swap(t.app[0], t.app[1]);
    if (!same_tensor(t.cast[0]->in[0], t.rope[1]->out) || !same_tensor(t.app[0]->in[0], t.cast[0]->out) || !same_tensor(t.app[1]->in[0], t.cast[1]->out))
        return false;
    if (same_tensor(t.cast[1]->in[0], t.rope[0]->out)) return false;          // v's cast reads no rope
    for (const aionhip_step *n : norm) {
        if (!n) continue;
        if (same_tensor(n->out, t.rope[0]->in[0])) t.norm[0] = n;
        else if (same_tensor(n->out, t.rope[1]->in[0])) t.norm[1] = n;
        else if (same_tensor(n->out, t.cast[1]->in[0])) t.norm[2] = n;
    }
    if (norms && (!t.norm[0] || !t.norm[1] || !t.norm[2])) return false;
    // one positions tensor and one set of RoPE parameters, one write index, f16 caches of one policy that do not overlap
    const aionhip_tensor_ref &kc = t.app[0]->out, &vc = t.app[1]->out;
    return t.rope[0]->in[1].handle == t.rope[1]->in[1].handle && t.rope[0]->rope_base == t.rope[1]->rope_base &&
           t.rope[0]->rope_scale == t.rope[1]->rope_scale && t.rope[0]->rope_proportion == t.rope[1]->rope_proportion &&
           t.app[0]->in[1].handle == t.app[1]->in[1].handle && kc.dtype == AIONHIP_F16 && vc.dtype == AIONHIP_F16 &&
           kc.shape[1] == vc.shape[1] && ((kc.flags ^ vc.flags) & AIONHIP_TENSOR_ROLLING) == 0 && !range_of(kc).overlaps(range_of(vc));
}

}  // namespace

int aionhip_session::check(size_t i, const aionhip_step &st) {
    auto bad = [&](const char *why) { return fail(i, st, AIONHIP_INVALID_ARGUMENT, why); };
    auto unsupported = [&](const char *why) { return fail(i, st, AIONHIP_UNSUPPORTED, why); };
    if (st.out.rank > AIONHIP_MAX_RANK) return bad("rank above 8");
    for (int j = 0; j < 5; ++j)
        if (st.in[j].rank > AIONHIP_MAX_RANK) return bad("rank above 8");
    switch (st.tag) {
    case AIONHIP_STEP_MATMUL:
    case AIONHIP_STEP_MATMUL_NT: {
        const aionhip_tensor_ref &a = st.in[0], &b = st.in[1], &c = st.out;
        if (!is_f32(a) || !is_f32(c) || !b.handle) return bad("MatMul: a and c are f32 device tensors, b a device tensor");
        if (b.rank != 2 || a.rank < 1 || c.rank != a.rank) return bad("MatMul: b is rank 2, c has a's rank");
        const bool nt = st.tag == AIONHIP_STEP_MATMUL_NT;
        const size_t n = nt ? b.shape[0] : b.shape[1], k = nt ? b.shape[1] : b.shape[0];
        if (a.shape[a.rank - 1] != k || c.shape[c.rank - 1] != n || rows_of(a) != rows_of(c)) return bad("MatMul: operand shapes do not agree");
        if (nt ? (b.dtype != AIONHIP_Q8_0 && b.dtype != AIONHIP_F32) : (b.dtype != AIONHIP_Q8_0 && b.dtype != AIONHIP_Q4_0))
            return unsupported(nt ? "MatMulNT: b is q8_0 or f32" : "MatMul: b is q4_0 or q8_0 (an f32 [K,N] operand stays on the CPU)");
        if (b.dtype != AIONHIP_F32 && k % 32 != 0) return bad("MatMul: the quantized axis is a whole number of 32-element blocks");
        if (!n || !k) return bad("MatMul: empty weight");
        return AIONHIP_OK;
    }
    case AIONHIP_STEP_ELEMWISE_BINARY: {
        const aionhip_tensor_ref &a = st.in[0], &b = st.in[1];
        if (!a.handle || !b.handle || !st.out.handle) return bad("ElemwiseBinary: null operand");
        if (a.dtype == AIONHIP_I32) {
            if (st.op != AIONHIP_BINARY_ADD || st.broadcast != 0 || !is_i32(b) || !is_i32(st.out)) return unsupported("ElemwiseBinary on i32: same-shape add only");
            if (elems(a) != elems(st.out) || elems(b) != elems(st.out)) return bad("ElemwiseBinary: identical broadcast needs equal sizes");
            return AIONHIP_OK;
        }
        if (!is_f32(a) || !is_f32(b) || !is_f32(st.out)) return unsupported("ElemwiseBinary: f32 or i32 operands");
        if (elems(a) != elems(st.out)) return unsupported("ElemwiseBinary: a has the output's shape");
        if (st.op == AIONHIP_BINARY_GATE) {
            if (st.act != AIONHIP_UNARY_GELU || st.broadcast != 0) return unsupported("gate: gelu, no broadcast");
            if (elems(b) != elems(st.out)) return bad("gate: operands of one shape");
            return AIONHIP_OK;
        }
        if (st.op < AIONHIP_BINARY_ADD || st.op > AIONHIP_BINARY_DIV) return unsupported("ElemwiseBinary: add, sub, mul, div or gate");
        if (st.broadcast == 0) { if (elems(b) != elems(st.out)) return bad("ElemwiseBinary: identical broadcast needs equal sizes"); }
        else if (st.broadcast == 2) { if (elems(b) != 1) return bad("ElemwiseBinary: scalar_b needs a one-element b"); }
        else if (st.broadcast == 4) { if (elems(b) == 0 || elems(st.out) % elems(b)) return bad("ElemwiseBinary: b is no suffix of the output's shape"); }
        else return unsupported("ElemwiseBinary: identical, scalar_b or contiguous_suffix_b broadcast");
        return AIONHIP_OK;
    }
    case AIONHIP_STEP_UNARY:
        if (!is_f32(st.in[0]) || !is_f32(st.out) || elems(st.in[0]) != elems(st.out)) return bad("Unary: f32 in and out of one size");
        if (st.op < AIONHIP_UNARY_RELU || st.op > AIONHIP_UNARY_SQRT) return unsupported("Unary: relu, gelu, silu, sigmoid, tanh or sqrt");
        return AIONHIP_OK;
    case AIONHIP_STEP_RMSNORM: {
        const aionhip_tensor_ref &x = st.in[0], &g = st.in[1], &be = st.in[2], &res = st.in[3];
        if (!is_f32(x) || !is_f32(g) || !is_f32(st.out)) return bad("RMSNorm: f32 x, gamma, out");
        const size_t cols = elems(g);
        if (cols == 0 || x.rank < 1 || x.shape[x.rank - 1] != cols || elems(x) != elems(st.out)) return bad("RMSNorm: gamma spans x's last axis");
        if (be.handle && (!is_f32(be) || elems(be) != cols)) return bad("RMSNorm: beta like gamma");
        if (res.handle && (!is_f32(res) || elems(res) != elems(x))) return bad("RMSNorm: residual like x");
        if (!(st.eps > 0.f) || !(st.eps < INFINITY)) return bad("RMSNorm: eps positive and finite");
        return AIONHIP_OK;
    }
    case AIONHIP_STEP_ATTENTION: {
        const aionhip_tensor_ref &q = st.in[0], &k = st.in[1], &v = st.in[2];
        if (!q.handle || !k.handle || !v.handle || !is_f32(st.out)) return bad("Attention: q, k, v and an f32 out");
        if (q.rank != 4 || k.rank != 4 || v.rank != 4 || st.out.rank != 4) return bad("Attention: rank-4 operands");
        if (k.dtype != v.dtype) return bad("Attention: k and v of one type");
        if (k.shape[0] != q.shape[0] || v.shape[0] != q.shape[0] || k.shape[3] != q.shape[3] || v.shape[1] != k.shape[1] || v.shape[2] != k.shape[2])
            return bad("Attention: operand shapes do not agree");
        if (st.out.shape[0] != q.shape[0] || st.out.shape[1] != q.shape[1] || st.out.shape[2] != q.shape[2] || st.out.shape[3] != v.shape[3])
            return bad("Attention: out is [B, L, Hq, Dv]");
        if (st.in[3].handle && (!is_i32(st.in[3]) || elems(st.in[3]) != q.shape[0] * q.shape[1])) return bad("Attention: query_positions i32 [B, L]");
        if (st.in[4].handle && (!is_i32(st.in[4]) || elems(st.in[4]) != q.shape[0])) return bad("Attention: kv_lengths i32 [B]");
        for (const aionhip_tensor_ref *t : {&q, &k})
            if (t->dtype != AIONHIP_F32 && t->dtype != AIONHIP_F16 && t->dtype != AIONHIP_BF16) return unsupported("Attention: f32, f16 or bf16 operands");
        if (k.shape[2] == 0 || q.shape[2] % k.shape[2] != 0) return bad("Attention: query heads are a multiple of the kv heads");
        return AIONHIP_OK;
    }
    case AIONHIP_STEP_ARGMAX: {
        const aionhip_tensor_ref &a = st.in[0];
        if (!is_f32(a) || !is_i32(st.out) || a.rank < 1) return bad("ArgMax: f32 in, i32 out");
        if (st.axis + 1 != (int)a.rank) return unsupported("ArgMax: over the last axis");
        if (elems(st.out) != rows_of(a)) return bad("ArgMax: out has one index per row");
        return AIONHIP_OK;
    }
    case AIONHIP_STEP_COPY:
        if (bytes_of(st.out) == 0 && elems(st.out) != 0) return unsupported("Copy: an element type this device does not hold");
        if (!st.in[0].handle || !st.out.handle || bytes_of(st.in[0]) != bytes_of(st.out) || st.in[0].dtype != st.out.dtype) return bad("Copy: src and dst of one type and size");
        return AIONHIP_OK;
    case AIONHIP_STEP_GATHER:
        if (st.axis != 0 || st.batch_dims != 0) return unsupported("Gather: axis 0 without batch dims");
        [[fallthrough]];
    case AIONHIP_STEP_GATHER_ROWS: {
        const aionhip_tensor_ref &t = st.in[0], &ids = st.in[1];
        if (!t.handle || t.rank != 2) return unsupported("Gather: a rank-2 table");
        if (t.dtype != AIONHIP_F32 && t.dtype != AIONHIP_Q8_0) return unsupported("Gather: an f32 or q8_0 table");
        if (!is_i32(ids) || !is_f32(st.out) || elems(st.out) != elems(ids) * t.shape[1]) return bad("Gather: i32 indices, f32 out [indices..., D]");
        if (t.dtype == AIONHIP_Q8_0 && t.shape[1] % 32 != 0) return bad("Gather: a q8_0 row is a whole number of 32-element blocks");
        return AIONHIP_OK;
    }
    case AIONHIP_STEP_ROPE1D: {
        const aionhip_tensor_ref &x = st.in[0], &pos = st.in[1];
        if (!is_f32(x) || !is_f32(st.out) || x.rank != 4 || elems(x) != elems(st.out)) return bad("RoPE1D: f32 [B, T, H, D] in and out");
        if (!is_i32(pos) || elems(pos) != x.shape[0] * x.shape[1]) return bad("RoPE1D: positions i32 [B, T]");
        if (x.shape[3] % 2 != 0 || x.shape[3] > 65534 || x.shape[2] > 65535) return bad("RoPE1D: an even head size");
        if (!(st.rope_base > 0.f) || !(st.rope_base < INFINITY) || !(st.rope_scale > 0.f) || !(st.rope_scale < INFINITY) ||
            !(st.rope_proportion >= 0.f && st.rope_proportion <= 1.f))
            return bad("RoPE1D: base and scale positive and finite, proportion in [0, 1]");
        return AIONHIP_OK;
    }
    case AIONHIP_STEP_SEQUENCE_APPEND: {
        const aionhip_tensor_ref &cache = st.out, &nk = st.in[0], &end = st.in[1];
        if (!cache.handle || !nk.handle || cache.rank != 4 || nk.rank != 4) return bad("SequenceAppend: rank-4 cache and rows");
        if (cache.dtype != nk.dtype) return bad("SequenceAppend: cache and rows of one type");
        if (cache.dtype != AIONHIP_F16 && cache.dtype != AIONHIP_F32) return unsupported("SequenceAppend: an f16 or f32 cache");
        if (cache.shape[0] != nk.shape[0] || cache.shape[2] != nk.shape[2] || cache.shape[3] != nk.shape[3]) return bad("SequenceAppend: rows are [B, S, H, D] of the cache's B, H, D");
        if (!is_i32(end) || elems(end) != cache.shape[0]) return bad("SequenceAppend: end_index i32 [B]");
        return AIONHIP_OK;
    }
    case AIONHIP_STEP_CAST:
        if (!is_f32(st.in[0]) || !st.out.handle || st.out.dtype != AIONHIP_F16) return unsupported("Cast: f32 to f16");
        if (elems(st.in[0]) != elems(st.out)) return bad("Cast: in and out of one size");
        return AIONHIP_OK;
    case AIONHIP_STEP_TRANSFER: {
        const aionhip_tensor_ref &dev = st.to_host ? st.in[0] : st.out;
        if (!dev.handle || !st.host) return bad("Transfer: a device tensor and host bytes");
        if (bytes_of(dev) == 0 && elems(dev) != 0) return unsupported("Transfer: an element type this device does not hold");
        if (st.host_bytes != bytes_of(dev)) return bad("Transfer: host bytes differ from the tensor's size");
        if (ctx->capturing) return bad("Transfer: not inside a recording");
        return AIONHIP_OK;
    }
    default:
        return unsupported("this device does not run the tag");
    }
}

int aionhip_session::check_list(const aionhip_step *steps, size_t count) {
    for (size_t i = 0; i < count; ++i) {
        const int rc = check(i, steps[i]);
        if (rc) return rc;
    }
    return AIONHIP_OK;
}

int aionhip_session::run_one(size_t i, const aionhip_step &st) {
    int rc = AIONHIP_OK;
    switch (st.tag) {
    case AIONHIP_STEP_MATMUL:
    case AIONHIP_STEP_MATMUL_NT: {
        const bool nt = st.tag == AIONHIP_STEP_MATMUL_NT;
        aionhip_weight *w = nullptr;
        rc = weight_for(st.in[1], nt ? AIONHIP_ROWS_NK : AIONHIP_KMAJOR_KN, &w);
        if (rc) break;
        rc = (nt ? aionhip_step_matmul_nt : aionhip_step_matmul)(ctx, w, rows_of(st.in[0]), st.in[0].handle, 0, st.out.handle, 0, st.alpha, st.beta);
        break;
    }
    case AIONHIP_STEP_ELEMWISE_BINARY: {
        const size_t n = elems(st.out);
        if (st.in[0].dtype == AIONHIP_I32) rc = aionhip_step_add_i32(ctx, st.out.handle, st.in[0].handle, st.in[1].handle, n);
        else if (st.op == AIONHIP_BINARY_GATE) rc = aionhip_step_gate_gelu(ctx, st.out.handle, st.in[0].handle, st.in[1].handle, n);
        else rc = aionhip_step_binary(ctx, st.op, st.out.handle, st.in[0].handle, st.in[1].handle, n, st.broadcast == 0 ? n : elems(st.in[1]));
        break;
    }
    case AIONHIP_STEP_UNARY:
        rc = aionhip_step_unary(ctx, st.op, st.out.handle, st.in[0].handle, elems(st.out));
        break;
    case AIONHIP_STEP_RMSNORM: {
        const size_t cols = elems(st.in[1]);
        rc = aionhip_step_rmsnorm(ctx, st.out.handle, st.in[0].handle, st.in[1].handle, st.in[2].handle, st.in[3].handle, elems(st.out) / cols, cols, st.eps);
        break;
    }
    case AIONHIP_STEP_ATTENTION: {
        const aionhip_tensor_ref &q = st.in[0], &k = st.in[1], &v = st.in[2];
        aionhip_attention p;
        memset(&p, 0, sizeof p);
        p.out = st.out.handle; p.q = q.handle; p.k = k.handle; p.v = v.handle;
        p.query_positions = st.in[3].handle; p.kv_lengths = st.in[4].handle;
        p.batch = q.shape[0]; p.l_q = q.shape[1]; p.h_q = q.shape[2]; p.d_k = q.shape[3];
        p.t_kv = k.shape[1]; p.h_kv = k.shape[2]; p.d_v = v.shape[3];
        p.q_dtype = q.dtype; p.kv_dtype = k.dtype;
        p.scale = st.scale; p.attn_logits_soft_cap = st.soft_cap;
        p.window_left = st.window_left; p.window_right = st.window_right; p.window_chunk = st.window_chunk;
        p.rolling = (k.flags & AIONHIP_TENSOR_ROLLING) ? 1 : 0;
        rc = aionhip_step_attention(ctx, &p);
        break;
    }
    case AIONHIP_STEP_ARGMAX: {
        const size_t n = st.in[0].shape[st.in[0].rank - 1];
        rc = aionhip_step_argmax(ctx, st.out.handle, st.in[0].handle, rows_of(st.in[0]), n);
        break;
    }
    case AIONHIP_STEP_COPY:
        rc = aionhip_d2d(ctx, st.out.handle, 0, st.in[0].handle, 0, bytes_of(st.out));
        break;
    case AIONHIP_STEP_GATHER:
    case AIONHIP_STEP_GATHER_ROWS:
        rc = aionhip_step_gather_rows(ctx, st.in[0].dtype, st.out.handle, st.in[0].handle, st.in[1].handle, elems(st.in[1]), st.in[0].shape[1], st.in[0].shape[0]);
        break;
    case AIONHIP_STEP_ROPE1D: {
        const aionhip_tensor_ref &x = st.in[0];
        rc = aionhip_step_rope(ctx, st.out.handle, x.handle, st.in[1].handle, x.shape[0], x.shape[1], x.shape[2], x.shape[3], st.rope_base, st.rope_scale, st.rope_proportion);
        break;
    }
    case AIONHIP_STEP_SEQUENCE_APPEND: {
        const aionhip_tensor_ref &cache = st.out, &nk = st.in[0];
        rc = aionhip_step_sequence_append(ctx, cache.dtype, cache.handle, nk.handle, st.in[1].handle, cache.shape[0], nk.shape[1], cache.shape[1],
                                          cache.shape[2] * cache.shape[3], (cache.flags & AIONHIP_TENSOR_ROLLING) ? 1 : 0);
        break;
    }
    case AIONHIP_STEP_CAST:
        rc = aionhip_step_cast_f32_f16(ctx, st.out.handle, st.in[0].handle, elems(st.out));
        break;
    case AIONHIP_STEP_TRANSFER:
        rc = st.to_host ? aionhip_d2h(ctx, st.host, st.in[0].handle, 0, st.host_bytes) : aionhip_h2d(ctx, st.out.handle, 0, st.host, st.host_bytes);
        break;
    default:
        return fail(i, st, AIONHIP_UNSUPPORTED, "this device does not run the tag");
    }
    ++calls_last_execute;
    return wrap(i, st, rc);
}

bool aionhip_session::only_read_within(const aionhip_step *steps, size_t count, size_t last, const aionhip_tensor_ref &t) const {
    if (!(t.flags & AIONHIP_TENSOR_WORKSPACE)) return false;
    const Range r = range_of(t);
    for (size_t j = last + 1; j < count; ++j) {
        if (reads_range(steps[j], r)) return false;
        if (writes_range(steps[j], r)) {
            // a step that overwrites the whole tensor ends the value's life; a partial write leaves part of it readable
            const Range w = range_of(steps[j].out);
            if (w.lo <= r.lo && w.hi >= r.hi) return true;
        }
    }
    return true;
}

aionhip_handle aionhip_session::residual_target(const aionhip_step *steps, size_t count, size_t j) const {
    if (!(fusion & AIONHIP_FUSE_WORKSPACE) || j + 1 >= count) return 0;
    const aionhip_step &mm = steps[j], &add = steps[j + 1];
    if (!is_matmul_tag(mm.tag) || mm.beta != 0.f) return 0;
    if (add.tag != AIONHIP_STEP_ELEMWISE_BINARY || add.op != AIONHIP_BINARY_ADD || add.broadcast != 0 || add.in[0].dtype != AIONHIP_F32) return 0;
    const aionhip_tensor_ref &t = mm.out;
    const aionhip_tensor_ref *x = same_tensor(add.in[1], t) ? &add.in[0] : same_tensor(add.in[0], t) ? &add.in[1] : nullptr;
    if (!x || !same_tensor(add.out, *x)) return 0;
    if (range_of(*x).overlaps(range_of(t)) || range_of(*x).overlaps(range_of(mm.in[0])) || range_of(*x).overlaps(range_of(mm.in[1]))) return 0;
    if (!only_read_within(steps, count, j + 1, t)) return 0;
    return x->handle;
}

// A pattern starting at step i run as one call: returns the number of steps consumed (0 = none matched, run step i alone).
// Every pattern's entry point gives the separate steps' results to the bit; one that answers AIONHIP_UNSUPPORTED has
// launched nothing, and the steps then run one by one.
size_t aionhip_session::try_fused(const aionhip_step *steps, size_t count, size_t i, int *rc_out) {
    const aionhip_step &st = steps[i];
    *rc_out = AIONHIP_OK;
    auto sibling_run = [&](size_t first, const aionhip_tensor_ref &a, const aionhip_weight **ws, aionhip_handle *cs) -> size_t {
        // MatMul / MatMulNT steps from `first` on that read exactly `a` with one alpha / beta and weights sharing k and dtype
        size_t c = 0;
        while (first + c < count && c < 4) {
            const aionhip_step &m = steps[first + c];
            if (!is_matmul_tag(m.tag) || !same_tensor(m.in[0], a) || m.in[1].dtype == AIONHIP_F32) break;
            if (c && (m.alpha != steps[first].alpha || m.beta != steps[first].beta || m.in[1].dtype != steps[first].in[1].dtype)) break;
            // a sibling may not write what a later sibling reads (its A), nor what an earlier one wrote
            bool clash = range_of(m.out).overlaps(range_of(a));
            for (size_t p = 0; p < c; ++p) clash |= range_of(m.out).overlaps(range_of(steps[first + p].out));
            if (clash) break;
            aionhip_weight *w = nullptr;
            if (weight_for(m.in[1], m.tag == AIONHIP_STEP_MATMUL_NT ? AIONHIP_ROWS_NK : AIONHIP_KMAJOR_KN, &w)) break;
            ws[c] = w;
            cs[c] = m.out.handle;
            ++c;
        }
        return c;
    };
    const aionhip_weight *ws[4];
    aionhip_handle cs[4];
    // A folded call reads the pattern's first inputs while (or after) it writes the pattern's outputs, where the separate steps
    // had finished with those inputs before the first output was written: no output may lie over such an input.
    auto clear_of = [&](const aionhip_tensor_ref &out, std::initializer_list<const aionhip_tensor_ref *> inputs) {
        for (const aionhip_tensor_ref *in : inputs)
            if (in->handle && range_of(out).overlaps(range_of(*in))) return false;
        return true;
    };
    auto siblings_clear_of = [&](size_t first, size_t c, std::initializer_list<const aionhip_tensor_ref *> inputs) {
        for (size_t m = 0; m < c; ++m)
            if (!clear_of(steps[first + m].out, inputs)) return false;
        return true;
    };

    auto dead_after = [&](const aionhip_tensor_ref &t, size_t last) { return only_read_within(steps, count, last, t); };
    const bool one_row = st.tag == AIONHIP_STEP_RMSNORM && !st.in[3].handle && elems(st.in[1]) == elems(st.out);

    // outputs of a folded cache side (rotated q, the two caches) clear of everything the fold reads, and of each other
    auto tail_outputs_clear = [&](const KvTail &t, std::initializer_list<const aionhip_tensor_ref *> inputs) {
        const aionhip_tensor_ref &qo = t.rope[0]->out, &kc = t.app[0]->out, &vc = t.app[1]->out;
        for (const aionhip_tensor_ref *o : {&qo, &kc, &vc})
            if (!clear_of(*o, inputs) || !clear_of(*o, {&t.rope[0]->in[1], &t.app[0]->in[1]})) return false;
        return !range_of(kc).overlaps(range_of(qo)) && !range_of(vc).overlaps(range_of(qo));
    };

    // One token of one sequence, the input side of an attention block: RMSNorm -> the q, k, v MatMuls -> RoPE1D on q and k ->
    // Cast f16 + SequenceAppend of k and of v (the six steps behind the matmuls in any order a valid program can have them)
    if ((fusion & AIONHIP_FUSE_WORKSPACE) && one_row && i + 9 < count && sibling_run(i + 1, st.out, ws, cs) == 3 &&
        steps[i + 1].alpha == 1.f && steps[i + 1].beta == 0.f) {
        KvTail t;
        if (sort_kv_tail(steps, i + 4, i + 10, 0, t)) {
            int iq = -1, ik = -1, iv = -1;
            for (int m = 0; m < 3; ++m) {
                const aionhip_tensor_ref &o = steps[i + 1 + m].out;
                if (same_tensor(o, t.rope[0]->in[0])) iq = m;
                else if (same_tensor(o, t.rope[1]->in[0])) ik = m;
                else if (same_tensor(o, t.cast[1]->in[0])) iv = m;
            }
            const aionhip_tensor_ref &xq = t.rope[0]->in[0], &xk = t.rope[1]->in[0], &kc = t.app[0]->out, &vc = t.app[1]->out;
            const size_t d = xq.shape[3];
            bool ok = iq >= 0 && ik >= 0 && iv >= 0 && xq.shape[0] == 1 && xq.shape[1] == 1 && xk.shape[0] == 1 && xk.shape[1] == 1 &&
                      xk.shape[3] == d && d % 8 == 0 && kc.shape[0] == 1 && vc.shape[0] == 1 && kc.shape[2] == xk.shape[2] &&
                      vc.shape[2] == xk.shape[2] && kc.shape[3] == d && vc.shape[3] == d &&
                      tail_outputs_clear(t, {&st.in[0], &st.in[1], &st.in[2]});
            // everything between the block's input and {rotated q, the caches} lives only inside these ten steps
            ok = ok && dead_after(st.out, i + 9) && dead_after(steps[i + 1].out, i + 9) && dead_after(steps[i + 2].out, i + 9) &&
                 dead_after(steps[i + 3].out, i + 9) && dead_after(t.rope[1]->out, i + 9) && dead_after(t.cast[0]->out, i + 9) &&
                 dead_after(t.cast[1]->out, i + 9);
            if (ok) {
                const int rc = aionhip_step_rmsnorm_qkv_rope_append(
                    ctx, ws[iq], ws[ik], ws[iv], st.in[0].handle, st.in[1].handle, st.in[2].handle, st.eps, t.rope[0]->out.handle, kc.handle, vc.handle,
                    t.rope[0]->in[1].handle, t.app[0]->in[1].handle, kc.shape[1], xq.shape[2], xk.shape[2], d, t.rope[0]->rope_base,
                    t.rope[0]->rope_scale, t.rope[0]->rope_proportion, (kc.flags & AIONHIP_TENSOR_ROLLING) ? 1 : 0);
                if (rc != AIONHIP_UNSUPPORTED) { *rc_out = wrap(i, st, rc); ++calls_last_execute; return 10; }
            }
        }
    }
    // Models that normalize their heads (src/bench/models.zig:455-473): RMSNorm over the head size on q, k and v -> RoPE1D on q and
    // k -> Cast f16 + SequenceAppend of k and of v, nine steps from the first of the norms on, in any order a valid program can
    // have them, for any batch and token count
    if ((fusion & AIONHIP_FUSE_WORKSPACE) && st.tag == AIONHIP_STEP_RMSNORM && !st.in[3].handle && st.in[0].rank == 4 &&
        elems(st.in[1]) == st.in[0].shape[3] && i + 8 < count) {
        KvTail t;
        if (sort_kv_tail(steps, i, i + 9, 3, t)) {
            const aionhip_step *nq = t.norm[0], *nk = t.norm[1], *nv = t.norm[2];
            const aionhip_tensor_ref &xq = nq->in[0], &xk = nk->in[0], &xv = nv->in[0], &kc = t.app[0]->out, &vc = t.app[1]->out;
            const size_t d = xq.shape[3];
            bool ok = xq.rank == 4 && xk.rank == 4 && xv.rank == 4 && xk.shape[3] == d && xv.shape[3] == d && xk.shape[0] == xq.shape[0] &&
                      xv.shape[0] == xq.shape[0] && xk.shape[1] == xq.shape[1] && xv.shape[1] == xq.shape[1] && xv.shape[2] == xk.shape[2] &&
                      elems(nq->in[1]) == d && elems(nk->in[1]) == d && elems(nv->in[1]) == d && nq->eps == nk->eps && nq->eps == nv->eps &&
                      kc.shape[0] == xq.shape[0] && vc.shape[0] == xq.shape[0] && kc.shape[2] == xk.shape[2] && vc.shape[2] == xk.shape[2] &&
                      kc.shape[3] == d && vc.shape[3] == d &&
                      tail_outputs_clear(t, {&xq, &xk, &xv, &nq->in[1], &nq->in[2], &nk->in[1], &nk->in[2], &nv->in[1], &nv->in[2]});
            ok = ok && dead_after(nq->out, i + 8) && dead_after(nk->out, i + 8) && dead_after(nv->out, i + 8) && dead_after(t.rope[1]->out, i + 8) &&
                 dead_after(t.cast[0]->out, i + 8) && dead_after(t.cast[1]->out, i + 8);
            if (ok) {
                const int rc = aionhip_step_headnorm_rope_append(
                    ctx, t.rope[0]->out.handle, xq.handle, xk.handle, xv.handle, nq->in[1].handle, nq->in[2].handle, nk->in[1].handle, nk->in[2].handle,
                    nv->in[1].handle, nv->in[2].handle, nq->eps, kc.handle, vc.handle, t.rope[0]->in[1].handle, t.app[0]->in[1].handle, xq.shape[0],
                    xq.shape[1], kc.shape[1], xq.shape[2], xk.shape[2], d, t.rope[0]->rope_base, t.rope[0]->rope_scale, t.rope[0]->rope_proportion,
                    (kc.flags & AIONHIP_TENSOR_ROLLING) ? 1 : 0);
                if (rc != AIONHIP_UNSUPPORTED) { *rc_out = wrap(i, st, rc); ++calls_last_execute; return 9; }
            }
        }
    }
    // The cache side without head norms, for any batch and token count (a prompt, several sequences): RoPE1D on q and k -> Cast f16
    // + SequenceAppend of k and of v, six steps from the first of the ropes on, linear caches
    if ((fusion & AIONHIP_FUSE_WORKSPACE) && st.tag == AIONHIP_STEP_ROPE1D && i + 5 < count) {
        KvTail t;
        if (sort_kv_tail(steps, i, i + 6, 0, t)) {
            const aionhip_tensor_ref &xq = t.rope[0]->in[0], &xk = t.rope[1]->in[0], &xv = t.cast[1]->in[0], &kc = t.app[0]->out, &vc = t.app[1]->out;
            const size_t d = xq.shape[3];
            bool ok = xv.rank == 4 && xk.shape[3] == d && xv.shape[3] == d && xk.shape[0] == xq.shape[0] && xv.shape[0] == xq.shape[0] &&
                      xk.shape[1] == xq.shape[1] && xv.shape[1] == xq.shape[1] && xv.shape[2] == xk.shape[2] && is_f32(xv) &&
                      kc.shape[0] == xq.shape[0] && vc.shape[0] == xq.shape[0] && kc.shape[2] == xk.shape[2] && vc.shape[2] == xk.shape[2] &&
                      kc.shape[3] == d && vc.shape[3] == d && !(kc.flags & AIONHIP_TENSOR_ROLLING) && xq.shape[1] <= kc.shape[1] &&
                      tail_outputs_clear(t, {&xq, &xk, &xv});
            ok = ok && dead_after(t.rope[1]->out, i + 5) && dead_after(t.cast[0]->out, i + 5) && dead_after(t.cast[1]->out, i + 5);
            if (ok) {
                const int rc = aionhip_step_rope_append(ctx, t.rope[0]->out.handle, xq.handle, xk.handle, xv.handle, kc.handle, vc.handle,
                                                        t.rope[0]->in[1].handle, t.app[0]->in[1].handle, xq.shape[0], xq.shape[1], kc.shape[1],
                                                        xq.shape[2], xk.shape[2], d, t.rope[0]->rope_base, t.rope[0]->rope_scale,
                                                        t.rope[0]->rope_proportion);
                if (rc != AIONHIP_UNSUPPORTED) { *rc_out = wrap(i, st, rc); ++calls_last_execute; return 6; }
            }
        }
    }
    // One row through a GeGLU feed-forward block: RMSNorm -> gate and up MatMuls -> gate(gelu) -> down MatMul
    if ((fusion & AIONHIP_FUSE_WORKSPACE) && one_row && i + 4 < count && sibling_run(i + 1, st.out, ws, cs) == 2) {
        const aionhip_step &g = steps[i + 3], &down = steps[i + 4];
        bool ok = g.tag == AIONHIP_STEP_ELEMWISE_BINARY && g.op == AIONHIP_BINARY_GATE && g.in[0].dtype == AIONHIP_F32 &&
                  steps[i + 1].alpha == 1.f && steps[i + 1].beta == 0.f && is_matmul_tag(down.tag) && down.in[1].dtype != AIONHIP_F32 &&
                  same_tensor(down.in[0], g.out);
        int ig = -1;
        if (ok) {
            if (same_tensor(g.in[0], steps[i + 1].out) && same_tensor(g.in[1], steps[i + 2].out)) ig = 0;
            else if (same_tensor(g.in[0], steps[i + 2].out) && same_tensor(g.in[1], steps[i + 1].out)) ig = 1;
            // (the output may be the block's own input x: the first of the two launches has consumed x before the second writes)
            ok = ig >= 0 && dead_after(st.out, i + 4) && dead_after(steps[i + 1].out, i + 4) && dead_after(steps[i + 2].out, i + 4) &&
                 dead_after(g.out, i + 4) && clear_of(down.out, {&st.in[1], &st.in[2]});
        }
        aionhip_weight *wd = nullptr;
        if (ok && weight_for(down.in[1], down.tag == AIONHIP_STEP_MATMUL_NT ? AIONHIP_ROWS_NK : AIONHIP_KMAJOR_KN, &wd) == AIONHIP_OK) {
            // x = x + down(...) behind it: the block's own input may be the residual it is added to
            const aionhip_handle res = residual_target(steps, count, i + 4);
            const int rc = aionhip_step_rmsnorm_geglu_matmul(ctx, ws[ig], ws[1 - ig], wd, st.in[0].handle, st.in[1].handle, st.in[2].handle, st.eps,
                                                             res ? res : down.out.handle, down.alpha, res ? 1.f : down.beta);
            if (rc != AIONHIP_UNSUPPORTED) { *rc_out = wrap(i, st, rc); ++calls_last_execute; return res ? 6 : 5; }
        }
    }
    if ((fusion & AIONHIP_FUSE_WORKSPACE) && st.tag == AIONHIP_STEP_RMSNORM && !st.in[3].handle && i + 1 < count) {
        const size_t c = sibling_run(i + 1, st.out, ws, cs);
        if (c && only_read_within(steps, count, i + c, st.out) && siblings_clear_of(i + 1, c, {&st.in[0], &st.in[1], &st.in[2]})) {
            const size_t cols = elems(st.in[1]);
            const int rc = aionhip_step_rmsnorm_matmul(ctx, c, ws, elems(st.out) / cols, st.in[0].handle, st.in[1].handle, st.in[2].handle, st.eps, cs, nullptr,
                                                       steps[i + 1].alpha, steps[i + 1].beta);
            if (rc != AIONHIP_UNSUPPORTED) { *rc_out = wrap(i, st, rc); ++calls_last_execute; return 1 + c; }
        }
    }
    if ((fusion & AIONHIP_FUSE_WORKSPACE) && st.tag == AIONHIP_STEP_ELEMWISE_BINARY && st.op == AIONHIP_BINARY_GATE && st.in[0].dtype == AIONHIP_F32 &&
        i + 1 < count) {
        const size_t c = sibling_run(i + 1, st.out, ws, cs);
        if (c >= 1 && only_read_within(steps, count, i + 1, st.out) && clear_of(steps[i + 1].out, {&st.in[0], &st.in[1]})) {
            aionhip_handle res = residual_target(steps, count, i + 1);
            if (res && !clear_of(steps[i + 2].out, {&st.in[0], &st.in[1]})) res = 0;
            const int rc = aionhip_step_gate_matmul(ctx, ws[0], rows_of(st.out), st.in[0].handle, st.in[1].handle, res ? res : cs[0], 0, steps[i + 1].alpha,
                                                    res ? 1.f : steps[i + 1].beta);
            if (rc != AIONHIP_UNSUPPORTED) { *rc_out = wrap(i, st, rc); ++calls_last_execute; return res ? 3 : 2; }
        }
    }
    if ((fusion & AIONHIP_FUSE_WORKSPACE) && st.tag == AIONHIP_STEP_CAST && i + 1 < count) {
        const aionhip_step &ap = steps[i + 1];
        if (ap.tag == AIONHIP_STEP_SEQUENCE_APPEND && ap.out.dtype == AIONHIP_F16 && same_tensor(ap.in[0], st.out) &&
            !range_of(ap.out).overlaps(range_of(st.in[0])) && only_read_within(steps, count, i + 1, st.out)) {
            const aionhip_tensor_ref &cache = ap.out, &nk = ap.in[0];
            const int rc = aionhip_step_append_f16(ctx, cache.handle, st.in[0].handle, ap.in[1].handle, cache.shape[0], nk.shape[1], cache.shape[1],
                                                   cache.shape[2] * cache.shape[3], (cache.flags & AIONHIP_TENSOR_ROLLING) ? 1 : 0);
            if (rc != AIONHIP_UNSUPPORTED) { *rc_out = wrap(i, st, rc); ++calls_last_execute; return 2; }
        }
    }
    if (is_matmul_tag(st.tag) && st.in[1].dtype != AIONHIP_F32) {
        const aionhip_handle res = residual_target(steps, count, i);
        aionhip_weight *w = nullptr;
        if (res && weight_for(st.in[1], st.tag == AIONHIP_STEP_MATMUL_NT ? AIONHIP_ROWS_NK : AIONHIP_KMAJOR_KN, &w) == AIONHIP_OK) {
            const int rc = (st.tag == AIONHIP_STEP_MATMUL_NT ? aionhip_step_matmul_nt : aionhip_step_matmul)(ctx, w, rows_of(st.in[0]), st.in[0].handle, 0, res, 0,
                                                                                                             st.alpha, 1.f);
            *rc_out = wrap(i, st, rc);
            ++calls_last_execute;
            return 2;
        }
    }
    if ((fusion & AIONHIP_FUSE_SIBLINGS) && is_matmul_tag(st.tag)) {
        const size_t c = sibling_run(i, st.in[0], ws, cs);
        if (c >= 2) {
            const int rc = aionhip_step_matmul_batch(ctx, c, ws, rows_of(st.in[0]), st.in[0].handle, 0, cs, nullptr, st.alpha, st.beta);
            if (rc != AIONHIP_UNSUPPORTED) { *rc_out = wrap(i, st, rc); ++calls_last_execute; return c; }
        }
    }
    return 0;
}

extern "C" {

int aionhip_session_create(aionhip_ctx *ctx, aionhip_session **out) {
    if (!ctx || !out) return AIONHIP_INVALID_ARGUMENT;
    aionhip_session *s = new (std::nothrow) aionhip_session;
    if (!s) return set_err(ctx, AIONHIP_OUT_OF_MEMORY, "session: host allocation failed");
    s->ctx = ctx;
    *out = s;
    return AIONHIP_OK;
}

int aionhip_session_set_fusion(aionhip_session *s, int mask) {
    if (!s) return AIONHIP_INVALID_ARGUMENT;
    if (mask & ~(AIONHIP_FUSE_SIBLINGS | AIONHIP_FUSE_WORKSPACE)) return set_err(s->ctx, AIONHIP_INVALID_ARGUMENT, "session: unknown fusion bits");
    s->fusion = mask;
    return AIONHIP_OK;
}

int aionhip_session_execute(aionhip_session *s, const aionhip_step *steps, size_t count) {
    if (!s) return AIONHIP_INVALID_ARGUMENT;
    if (count && !steps) return set_err(s->ctx, AIONHIP_INVALID_ARGUMENT, "session: null step list");
    int rc = s->check_list(steps, count);
    if (rc) return rc;
    s->calls_last_execute = 0;
    for (size_t i = 0; i < count;) {
        const size_t used = s->fusion ? s->try_fused(steps, count, i, &rc) : 0;
        if (rc) return rc;
        if (used) { i += used; continue; }
        rc = s->run_one(i, steps[i]);
        if (rc) return rc;
        ++i;
    }
    return AIONHIP_OK;
}

int aionhip_session_stats(const aionhip_session *s, uint64_t *calls_last_execute, uint64_t *weights, uint64_t *weight_bytes) {
    if (!s) return AIONHIP_INVALID_ARGUMENT;
    if (calls_last_execute) *calls_last_execute = s->calls_last_execute;
    if (weights) *weights = s->weights.size();
    if (weight_bytes) {
        uint64_t b = 0;
        for (const auto &kv : s->weights) b += aionhip_weight_device_bytes(kv.second);
        *weight_bytes = b;
    }
    return AIONHIP_OK;
}

int aionhip_session_retire(aionhip_session *s) {
    if (!s) return AIONHIP_INVALID_ARGUMENT;
    const int rc = aionhip_sync(s->ctx);
    s->drop_weights();
    return rc;
}

void aionhip_session_destroy(aionhip_session *s) {
    if (!s) return;
    aionhip_session_retire(s);
    delete s;
}

}  // extern "C"
