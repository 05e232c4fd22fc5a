// Backend optimizer pass: recognises the exact instruction sequences the reference's functionals
// emit (crates/gpt-rs/src/ops/functional/*.rs) and rewrites each to one fused instruction.
// The reference's Triton backend does the same job with #[ptir_pattern] views
// (crates/gpt-rs-backend-triton/src/optimizer/layer_norm_fusion.rs:30-97); here the matcher runs
// inside the executor on the program it is handed, so it needs no front-end support.
//
// Matching is structural on the def-use graph, rooted at the last instruction of a sequence.
// A fused instruction takes over the root's value id; the sequence's interior instructions are
// left in place and removed by dead-code elimination when nothing else reads them, so a value the
// caller also asked for (e.g. layer_norm's mean) is still produced by the generic path.
#include <algorithm>
#include <cmath>
#include <array>
#include <cstring>
#include <map>

#include "kernels.hpp"
#include "runtime.hpp"

namespace gptrs {
namespace {

struct Fuser {
    Function& fn;
    std::vector<int> def;   // value id -> body index, -1 for parameters
    int fused = 0;

    explicit Fuser(Function& f) : fn(f) { reindex(); }

    void reindex() {
        def.assign(fn.max_value_id + 1, -1);
        for (size_t i = 0; i < fn.body.size(); ++i)
            if (!fn.body[i].dead)
                for (int id : fn.body[i].out_ids) def[id] = (int)i;
    }
    const Instr* producer(int v) const {
        if (v < 0 || v >= (int)def.size() || def[v] < 0) return nullptr;
        return &fn.body[def[v]];
    }
    const Spec* spec_of(int v) const {
        if (v < 0) return nullptr;
        if (const Instr* p = producer(v)) {
            for (size_t i = 0; i < p->out_ids.size(); ++i)
                if (p->out_ids[i] == v) return &p->out_specs[i];
            return nullptr;
        }
        for (size_t i = 0; i < fn.param_ids.size(); ++i)
            if (fn.param_ids[i] == v) return &fn.param_specs[i];
        return nullptr;
    }
    // Looks through instructions that do not change the value: identity Slice / BroadcastTo /
    // Transpose / Reshape-to-same-shape (the front end's canonicaliser removes these,
    // crates/gpt-rs/src/backend/pipeline.rs:74-119) and StopGradient.
    int strip(int v) const {
        for (;;) {
            const Instr* p = producer(v);
            if (!p || p->operands.empty() || p->operands[0].value < 0) return v;
            const Spec* in = spec_of(p->operands[0].value);
            if (!in) return v;
            bool ident = false;
            switch (p->op) {
                case OpKind::StopGradient: ident = true; break;
                case OpKind::Reshape: case OpKind::BroadcastTo: ident = in->dims == p->out_specs[0].dims; break;
                case OpKind::Slice:
                    ident = in->dims == p->out_specs[0].dims;
                    for (auto s : p->a) ident = ident && s == 0;
                    break;
                case OpKind::Transpose:
                    ident = true;
                    for (size_t i = 0; i < p->a.size(); ++i) ident = ident && p->a[i] == (int64_t)i;
                    break;
                default: break;
            }
            if (!ident) return v;
            v = p->operands[0].value;
        }
    }
    const Instr* prod(int v) const { return producer(strip(v)); }

    // ---- small matchers; every `v` is stripped first
    bool binary(int v, BinaryOp op, int& a, int& b) const {
        const Instr* p = prod(v);
        if (!p || p->op != OpKind::Binary || p->binary != op || p->scalar_rhs) return false;
        a = p->operands[0].value;
        b = p->operands[1].value;
        return a >= 0 && b >= 0;
    }
    bool unary(int v, UnaryOp op, int& a) const {
        const Instr* p = prod(v);
        if (!p || p->op != OpKind::Unary || p->unary != op) return false;
        a = p->operands[0].value;
        return a >= 0;
    }
    bool bcast(int v, int& src) const {  // a real (non-identity) broadcast of a value
        const Instr* p = prod(v);
        if (!p || p->op != OpKind::BroadcastTo) return false;
        src = p->operands[0].value;
        return src >= 0;
    }
    bool reduce_last(int v, ReduceKind kind, int& src) const {
        const Instr* p = prod(v);
        if (!p || p->op != OpKind::Reduce || p->reduce != kind || !p->keepdims || p->a.size() != 1) return false;
        src = p->operands[0].value;
        const Spec* s = spec_of(src);
        if (!s || s->rank() < 1) return false;
        int64_t ax = p->a[0] < 0 ? p->a[0] + s->rank() : p->a[0];
        return ax == s->rank() - 1;
    }
    static bool literal_scalar(const Literal& l, float& out) {
        if (l.spec.count() != 1) return false;
        if (l.spec.dtype == DType::F32) { memcpy(&out, l.bytes.data(), 4); return true; }
        if (l.spec.dtype == DType::BF16) {
            uint16_t b; memcpy(&b, l.bytes.data(), 2);
            uint32_t u = (uint32_t)b << 16; memcpy(&out, &u, 4); return true;
        }
        return false;
    }
    // BroadcastTo(...BroadcastTo(Literal scalar)) chains (crates/gpt-rs/src/ops/ptir/graph.rs:757-793)
    bool scalar(int v, float& out) const {
        for (int depth = 0; depth < 4; ++depth) {
            const Instr* p = producer(v);
            if (!p) return false;
            if (p->op == OpKind::Constant) return literal_scalar(fn.literals[p->literal], out);
            if (p->op != OpKind::BroadcastTo && p->op != OpKind::Reshape) return false;
            const Operand& o = p->operands[0];
            if (o.value < 0) return literal_scalar(fn.literals[o.literal], out);
            v = o.value;
        }
        return false;
    }
    // Add/Mul in either operand order: `pred(x)` picks which side is which
    template <typename F>
    bool binary_comm(int v, BinaryOp op, int& first, int& second, F is_second) const {
        int a, b;
        if (!binary(v, op, a, b)) return false;
        if (is_second(b)) { first = a; second = b; return true; }
        if (is_second(a)) { first = b; second = a; return true; }
        return false;
    }
    // BroadcastTo(x) along leading axes of a vector x of n values (shape [n] or [1, .., 1, n]).  A program INPUT of n
    // values and last extent n counts as the vector itself: that is what `BroadcastTo([1, n])(gamma)` has become when
    // the reference's optimizer has folded it into a derived parameter ahead of a one-row program
    // (crates/gpt-rs/src/backend/passes/param_only_fold_to_param.rs:24-160).
    bool vector_bcast_last(int v, int64_t n, int& vec) const {
        auto is_vector = [&](int q) {
            const Spec* s = spec_of(q);
            return s && s->rank() >= 1 && s->dims.back() == n && s->count() == n;
        };
        const int cur = strip(v);
        if (!producer(cur)) {   // a program input
            if (!is_vector(cur)) return false;
            vec = cur;
            return true;
        }
        int src;
        if (!bcast(cur, src)) return false;
        for (int depth = 0; depth < 4 && !is_vector(src); ++depth) {   // broadcasts of broadcasts (the canonicaliser collapses them)
            int inner;
            if (!bcast(src, inner)) return false;
            src = inner;
        }
        if (!is_vector(src)) return false;
        vec = src;
        return true;
    }
    bool slice(int v, int& src, std::vector<int64_t>& starts, std::vector<int64_t>& sizes) const {
        const Instr* p = producer(v);  // not stripped: identity slices are handled by callers via strip()
        if (!p || p->op != OpKind::Slice) return false;
        src = p->operands[0].value;
        starts = p->a;
        sizes = p->b;
        return src >= 0;
    }
    bool reshape_of(int v, int& src) const {
        const Instr* p = producer(v);
        if (!p || p->op != OpKind::Reshape) return false;
        src = p->operands[0].value;
        return src >= 0;
    }
    bool transpose102(int v, int& src) const {
        const Instr* p = producer(v);
        if (!p || p->op != OpKind::Transpose || p->a != std::vector<int64_t>{1, 0, 2}) return false;
        src = p->operands[0].value;
        return src >= 0;
    }

    // Replace the instruction that defines `root_v` by `ni` (placed where the root was).
    void replace_root(int root_v, Instr ni) {
        const int idx = def[root_v];
        ni.dead = false;
        fn.body[idx] = std::move(ni);
        ++fused;
    }
    void kill(int v) {  // mark the (non-root) producer of a secondary output dead
        if (def[v] >= 0) fn.body[def[v]].dead = true;
    }

    // The front end's canonicaliser collapses Slice(Slice(x)) (crates/gpt-rs/src/backend/passes/slice_canonicalization.rs:
    // 83-124): the rows of one sequence cut out of a stacked [B * T, P] projection and then its Q / K / V column blocks
    // arrive as single slices of the stacked tensor.  The patterns below are written over "a packed [T, P] tensor and
    // its column blocks", so such a slice is taken apart again: a row block (shared by the column blocks cut from it)
    // and a column block of it.  Row blocks nothing else reads cost nothing: the fused ops read through them.
    void pass_split_slices() {
        std::map<std::array<int64_t, 3>, int> row_block;   // (source, first row, rows) -> value
        std::vector<Instr> body;
        body.reserve(fn.body.size() + 16);
        bool changed = false;
        for (const Instr& in : fn.body) {
            if (!in.dead && in.op == OpKind::Slice && in.operands[0].value >= 0 && in.a.size() == 2) {
                const Spec* xs = spec_of(in.operands[0].value);
                if (xs && xs->rank() == 2 && in.b[0] < xs->dims[0] && in.b[1] < xs->dims[1]) {
                    const std::array<int64_t, 3> key{in.operands[0].value, in.a[0], in.b[0]};
                    auto it = row_block.find(key);
                    if (it == row_block.end()) {
                        Instr rb = make(OpKind::Slice, "Slice", {in.operands[0].value}, ++fn.max_value_id, Spec{xs->dtype, {in.b[0], xs->dims[1]}});
                        rb.a = {in.a[0], 0};
                        rb.b = {in.b[0], xs->dims[1]};
                        it = row_block.emplace(key, rb.out_ids[0]).first;
                        body.push_back(std::move(rb));
                    }
                    Instr cut = in;
                    cut.operands[0].value = it->second;
                    cut.a[0] = 0;
                    body.push_back(std::move(cut));
                    changed = true;
                    continue;
                }
            }
            body.push_back(in);   // (a copy: fn.body stays readable through spec_of while this loop runs)
        }
        if (changed) {
            fn.body = std::move(body);
            reindex();
        }
    }

    // ---------------------------------------------------------------- elementwise sequences
    bool m_softmax(int v, int& x) const {  // ops/functional/common.rs:22-31
        int e, sb, s, e2, sh, xx, mb, m, x2;
        if (!binary(v, BinaryOp::Div, e, sb)) return false;
        if (!bcast(sb, s) || !reduce_last(s, ReduceKind::Sum, e2) || strip(e2) != strip(e)) return false;
        if (!unary(e, UnaryOp::Exp, sh) || !binary(sh, BinaryOp::Sub, xx, mb)) return false;
        if (!bcast(mb, m) || !reduce_last(m, ReduceKind::Max, x2) || strip(x2) != strip(xx)) return false;
        x = xx;
        return true;
    }
    bool m_gelu(int v, int& x, float (&lit)[3]) const {  // activation.rs:96-113
        int half, op, xa, l0, er, l2, sc, xb, l1;
        if (!binary(v, BinaryOp::Mul, half, op)) return false;
        if (!binary(half, BinaryOp::Mul, xa, l0) || !scalar(l0, lit[0])) return false;
        if (!binary(op, BinaryOp::Add, er, l2) || !scalar(l2, lit[2])) return false;
        if (!unary(er, UnaryOp::Erf, sc) || !binary(sc, BinaryOp::Div, xb, l1) || !scalar(l1, lit[1])) return false;
        if (strip(xa) != strip(xb)) return false;
        x = xa;
        return true;
    }
    bool m_silu(int v, int& g) const {  // activation.rs:119-134
        int ga, d, e, l1, n, gb, lm;
        float one, neg;
        if (!binary(v, BinaryOp::Div, ga, d)) return false;
        if (!binary(d, BinaryOp::Add, e, l1) || !scalar(l1, one) || one != 1.0f) return false;
        if (!unary(e, UnaryOp::Exp, n) || !binary(n, BinaryOp::Mul, gb, lm) || !scalar(lm, neg) || neg != -1.0f) return false;
        if (strip(ga) != strip(gb)) return false;
        g = ga;
        return true;
    }
    bool m_layer_norm(int v, int& x, int& gamma, int& beta, float& inv_n, float& eps) const {  // normalization.rs:123-174
        const Spec* os = spec_of(v);
        if (!os || os->rank() < 1) return false;
        const int64_t n = os->dims.back();
        int t, bb, nrm, gb, cen, isb, is, ve, vm, eb, vs, ic, sq, c1, c2, xx, mb, mean, s, ic2, x2;
        float inv2;
        auto is_vec = [&](int q) { int tmp; return vector_bcast_last(q, n, tmp); };
        if (!binary_comm(v, BinaryOp::Add, t, bb, is_vec) || !vector_bcast_last(bb, n, beta)) return false;
        if (!binary_comm(t, BinaryOp::Mul, nrm, gb, is_vec) || !vector_bcast_last(gb, n, gamma)) return false;
        if (!binary(nrm, BinaryOp::Mul, cen, isb) || !bcast(isb, is) || !unary(is, UnaryOp::Rsqrt, ve)) return false;
        if (!binary(ve, BinaryOp::Add, vm, eb) || !scalar(eb, eps)) return false;
        if (!binary(vm, BinaryOp::Mul, vs, ic) || !scalar(ic, inv_n)) return false;
        if (!reduce_last(vs, ReduceKind::Sum, sq) || !binary(sq, BinaryOp::Mul, c1, c2)) return false;
        if (strip(c1) != strip(cen) || strip(c2) != strip(cen)) return false;
        if (!binary(cen, BinaryOp::Sub, xx, mb) || !bcast(mb, mean)) return false;
        if (!binary(mean, BinaryOp::Mul, s, ic2) || !scalar(ic2, inv2) || inv2 != inv_n) return false;
        if (!reduce_last(s, ReduceKind::Sum, x2) || strip(x2) != strip(xx)) return false;
        x = xx;
        return true;
    }
    bool m_rms_norm(int v, int& x, int& gamma, float& inv_n, float& eps) const {  // normalization.rs:183-217
        const Spec* os = spec_of(v);
        if (!os || os->rank() < 1) return false;
        const int64_t n = os->dims.back();
        int nrm, gb, xx, irb, ir, t, ms, eb, s, ic, sq, x1, x2;
        auto is_vec = [&](int q) { int tmp; return vector_bcast_last(q, n, tmp); };
        if (!binary_comm(v, BinaryOp::Mul, nrm, gb, is_vec) || !vector_bcast_last(gb, n, gamma)) return false;
        if (!binary(nrm, BinaryOp::Mul, xx, irb) || !bcast(irb, ir) || !unary(ir, UnaryOp::Rsqrt, t)) return false;
        if (!binary(t, BinaryOp::Add, ms, eb) || !scalar(eb, eps)) return false;
        if (!binary(ms, BinaryOp::Mul, s, ic) || !scalar(ic, inv_n)) return false;
        if (!reduce_last(s, ReduceKind::Sum, sq) || !binary(sq, BinaryOp::Mul, x1, x2)) return false;
        if (strip(x1) != strip(xx) || strip(x2) != strip(xx)) return false;
        x = xx;
        return true;
    }

    // Cast(bf16)(rms_norm(x f32, gamma f32)): the norm stores bf16 directly (one rounding of the f32 result, which is
    // what the cast does).  The reference's rms_norm is f32-only (normalization.rs:183-217), so a bf16 model with an
    // f32 residual stream reaches its bf16 projections through exactly this pair.
    void pass_norm_cast() {
        const std::vector<int> uses = count_uses();
        for (auto& in : fn.body) {
            if (in.dead || in.op != OpKind::Cast || in.out_specs[0].dtype != DType::BF16) continue;
            const int src = in.operands[0].value;
            if (src < 0 || def[src] < 0 || uses[src] != 1) continue;
            Instr& nrm = fn.body[def[src]];
            if (nrm.dead || nrm.op != OpKind::FRmsNorm || nrm.out_specs[0].dtype != DType::F32) continue;
            Instr ni = nrm;
            ni.out_ids = in.out_ids;
            ni.out_specs = in.out_specs;
            nrm.dead = true;
            in = ni;
            ++fused;
        }
        reindex();
    }

    Instr make(OpKind op, const char* name, std::vector<int> ins, int out_id, const Spec& out_spec) const {
        Instr ni;
        ni.op = op;
        ni.op_name = name;
        for (int v : ins) { Operand o; o.value = v; ni.operands.push_back(o); }
        ni.out_ids = {out_id};
        ni.out_specs = {out_spec};
        return ni;
    }

    // Roots are visited last-to-first so a larger sequence claims its instructions before a
    // smaller one nested inside it can (layer_norm contains an rms_norm-shaped tail; swiglu
    // contains silu).
    void pass_elementwise() {
        for (int i = (int)fn.body.size() - 1; i >= 0; --i) {
            Instr& in = fn.body[i];
            if (in.dead || in.op != OpKind::Binary || in.scalar_rhs) continue;
            const int v = in.out_ids[0];
            const Spec out = in.out_specs[0];
            if (!dtype_is_float(out.dtype)) continue;
            int x, g, b, u;
            float inv_n, eps, lit[3];
            if (in.binary == BinaryOp::Div && m_softmax(v, x)) {
                replace_root(v, make(OpKind::FSoftmax, "fused.softmax", {x}, v, out));
            } else if (in.binary == BinaryOp::Add && m_layer_norm(v, x, g, b, inv_n, eps)) {
                Instr ni = make(OpKind::FLayerNorm, "fused.layer_norm", {x, g, b}, v, out);
                ni.scale = inv_n; ni.eps = eps;
                replace_root(v, ni);
            } else if (in.binary == BinaryOp::Mul && m_rms_norm(v, x, g, inv_n, eps)) {
                Instr ni = make(OpKind::FRmsNorm, "fused.rms_norm", {x, g}, v, out);
                ni.scale = inv_n; ni.eps = eps;
                replace_root(v, ni);
            } else if (in.binary == BinaryOp::Mul && m_gelu(v, x, lit)) {
                Instr ni = make(OpKind::FGelu, "fused.gelu", {x}, v, out);
                ni.fparam[0] = lit[0]; ni.fparam[1] = lit[1]; ni.fparam[2] = lit[2];
                replace_root(v, ni);
            } else if (in.binary == BinaryOp::Mul) {
                int a = in.operands[0].value, c = in.operands[1].value;
                if (a >= 0 && c >= 0 && m_silu(a, g)) { u = c; replace_root(v, make(OpKind::FSwiglu, "fused.swiglu", {g, u}, v, out)); }
            } else if (in.binary == BinaryOp::Div && m_silu(v, g)) {
                replace_root(v, make(OpKind::FSilu, "fused.silu", {g}, v, out));
            }
        }
    }

    // ---------------------------------------------------------------- RoPE on packed QKV
    // rotary.rs:430-536.  Matches one head group: v == Reshape([T, H*Dh])(Transpose[1,0,2](rotated))
    bool m_rope_group(int v, int& qkv, int64_t& col, int64_t& heads, int64_t& dh, int64_t& half, int& cos, int& sin) const {
        int tr, rot;
        if (!reshape_of(strip(v), tr) || !transpose102(strip(tr), rot)) return false;
        rot = strip(rot);
        const Instr* cat = producer(rot);
        if (!cat || cat->op != OpKind::Concat || cat->axis != 2 || cat->operands.size() != 2) return false;
        int fr = cat->operands[0].value, sr = cat->operands[1].value;
        int pass = -1;
        {   // partial rotary: Concat(2)(Concat(2)(fr, sr), pass)
            const Instr* inner = producer(strip(fr));
            if (inner && inner->op == OpKind::Concat && inner->axis == 2 && inner->operands.size() == 2) {
                pass = sr;
                fr = inner->operands[0].value;
                sr = inner->operands[1].value;
            }
        }
        int m1, m2, m3, m4, a1, c1, b1, s1, b2, c2, a2, s2;
        if (!binary(fr, BinaryOp::Sub, m1, m2) || !binary(sr, BinaryOp::Add, m3, m4)) return false;
        if (!binary(m1, BinaryOp::Mul, a1, c1) || !binary(m2, BinaryOp::Mul, b1, s1)) return false;
        if (!binary(m3, BinaryOp::Mul, b2, c2) || !binary(m4, BinaryOp::Mul, a2, s2)) return false;
        if (strip(a1) != strip(a2) || strip(b1) != strip(b2) || strip(c1) != strip(c2) || strip(s1) != strip(s2)) return false;
        // a = Slice(xr,[0,0,0],[H,T,half]), b = Slice(xr,[0,0,half],[H,T,half])
        int xa, xb;
        std::vector<int64_t> st, sz, st2, sz2;
        if (!slice(strip(a1), xa, st, sz) || !slice(strip(b1), xb, st2, sz2)) return false;
        if (sz.size() != 3 || sz != sz2 || st != std::vector<int64_t>{0, 0, 0}) return false;
        heads = sz[0];
        const int64_t T = sz[1];
        half = sz[2];
        if (st2 != std::vector<int64_t>{0, 0, half}) return false;
        int xh = strip(xa);  // xr (identity slice when rotary_dim == head_dim) or a real slice of xh
        if (strip(xb) != xh) return false;
        {
            int src; std::vector<int64_t> s3, z3;
            if (slice(xh, src, s3, z3)) {
                if (s3 != std::vector<int64_t>{0, 0, 0} || z3 != std::vector<int64_t>{heads, T, 2 * half}) return false;
                xh = strip(src);
            }
        }
        const Spec* xs = spec_of(xh);
        if (!xs || xs->rank() != 3 || xs->dims[0] != heads || xs->dims[1] != T) return false;
        dh = xs->dims[2];
        if (2 * half > dh) return false;
        if (pass >= 0) {
            int ps; std::vector<int64_t> s4, z4;
            if (!slice(strip(pass), ps, s4, z4) || strip(ps) != xh) return false;
            if (s4 != std::vector<int64_t>{0, 0, 2 * half} || z4 != std::vector<int64_t>{heads, T, dh - 2 * half}) return false;
        } else if (2 * half != dh) {
            return false;
        }
        // xh = Transpose[1,0,2](Reshape([T,H,dh])(Slice(qkv,[0,col],[T,H*dh])))
        int rs, sl, q;
        std::vector<int64_t> s5, z5;
        if (!transpose102(xh, rs) || !reshape_of(strip(rs), sl)) return false;
        const Spec* rss = spec_of(strip(rs));
        if (!rss || rss->dims != std::vector<int64_t>{T, heads, dh}) return false;
        if (!slice(sl, q, s5, z5) || s5.size() != 2 || s5[0] != 0 || z5 != std::vector<int64_t>{T, heads * dh}) return false;
        qkv = q;
        col = s5[1];
        // cos/sin: BroadcastTo([H,T,half])(Reshape([1,T,half])(cos))
        auto table = [&](int cv, int& tab) {
            int r;
            const Instr* p = producer(strip(cv));
            if (!p) return false;
            if (p->op == OpKind::BroadcastTo) {
                if (p->out_specs[0].dims != std::vector<int64_t>{heads, T, half}) return false;
                r = p->operands[0].value;
            } else {
                r = strip(cv);  // heads == 1: the broadcast is an identity
            }
            if (r < 0) return false;
            int src;
            if (!reshape_of(strip(r), src)) return false;
            const Spec* ts = spec_of(src);
            if (!ts || ts->dims != std::vector<int64_t>{T, half}) return false;
            tab = src;
            return true;
        };
        return table(c1, cos) && table(s1, sin);
    }

    void pass_rope() {
        for (size_t i = 0; i < fn.body.size(); ++i) {
            Instr& in = fn.body[i];
            if (in.dead || in.op != OpKind::Concat || in.axis != 1 || in.operands.size() != 3) continue;
            const Spec out = in.out_specs[0];
            if (out.rank() != 2 || !dtype_is_float(out.dtype)) continue;
            const int qv = in.operands[0].value, kv = in.operands[1].value, vv = in.operands[2].value;
            if (qv < 0 || kv < 0 || vv < 0) continue;
            int qkv_q, qkv_k, cq, sq, ck, sk;
            int64_t colq, hq, dq, halfq, colk, hk, dk, halfk;
            if (!m_rope_group(qv, qkv_q, colq, hq, dq, halfq, cq, sq)) continue;
            if (!m_rope_group(kv, qkv_k, colk, hk, dk, halfk, ck, sk)) continue;
            if (qkv_q != qkv_k || cq != ck || sq != sk || dq != dk || halfq != halfk) continue;
            if (colq != 0 || colk != hq * dq) continue;
            int vsrc; std::vector<int64_t> s, z;
            if (!slice(strip(vv), vsrc, s, z) || vsrc != qkv_q) continue;
            const int64_t T = out.dims[0];
            if (s != std::vector<int64_t>{0, (hq + hk) * dq} || z != std::vector<int64_t>{T, hk * dq}) continue;
            const Spec* qs = spec_of(qkv_q);
            if (!qs || qs->dims != out.dims || out.dims[1] != (hq + 2 * hk) * dq) continue;
            Instr ni = make(OpKind::FRope, "fused.rope_qkv_packed", {qkv_q, cq, sq}, in.out_ids[0], out);
            ni.n_q = hq; ni.n_kv = hk; ni.head_dim = dq; ni.rot_half = halfq;
            replace_root(in.out_ids[0], ni);
        }
    }

    // ---------------------------------------------------------------- attention
    // Walks Reshape / BroadcastTo([Hkv,g,L,Dh]) / Reshape back to the [Hkv, L, Dh] source of a
    // grouped K or V operand (attention.rs:703-711).
    bool group_source(int v, int64_t hq, int64_t L, int64_t dh, int& src, int64_t& hkv) const {
        int64_t g = 1;
        for (int depth = 0; depth < 6; ++depth) {
            v = strip(v);
            const Spec* s = spec_of(v);
            if (!s) return false;
            const Instr* p = producer(v);
            if (p && p->op == OpKind::Reshape) { v = p->operands[0].value; if (v < 0) return false; continue; }
            if (p && p->op == OpKind::BroadcastTo) {
                const Spec* is = spec_of(p->operands[0].value);
                const Spec& os = p->out_specs[0];
                if (!is || os.rank() != 4 || is->rank() != 4 || is->dims[1] != 1 || is->dims[0] != os.dims[0] ||
                    is->dims[2] != L || is->dims[3] != dh || os.dims[2] != L || os.dims[3] != dh)
                    return false;
                g = os.dims[1];
                v = p->operands[0].value;
                continue;
            }
            if (s->rank() == 3 && s->dims[1] == L && s->dims[2] == dh && s->dims[0] * g == hq) {
                src = v;
                hkv = s->dims[0];
                return true;
            }
            return false;
        }
        return false;
    }
    bool is_dot(int v, std::vector<int64_t> bl, std::vector<int64_t> br, std::vector<int64_t> cl, std::vector<int64_t> cr,
                int& a, int& b) const {
        const Instr* p = producer(strip(v));
        if (!p || p->op != OpKind::Dot || p->a != bl || p->b != br || p->c != cl || p->d != cr) return false;
        a = p->operands[0].value;
        b = p->operands[1].value;
        return a >= 0 && b >= 0;
    }
    // select(qpos >= pos, 0, -big): returns the compare's operands
    bool m_mask_select(int v, int& lhs, int& rhs) const {
        const Instr* p = producer(strip(v));
        if (!p || p->op != OpKind::Select) return false;
        const Instr* c = producer(strip(p->operands[0].value));
        float z, ng;
        if (!c || c->op != OpKind::Compare || c->cmp != CmpOp::GreaterEqual) return false;
        if (p->operands[1].value < 0 || p->operands[2].value < 0) return false;
        if (!scalar(p->operands[1].value, z) || !scalar(p->operands[2].value, ng)) return false;
        // the kernels drop masked terms outright, exact only while exp(mask + s - max) underflows to 0
        if (z != 0.0f || !(ng <= -1e8f)) return false;
        lhs = c->operands[0].value;
        rhs = c->operands[1].value;
        return lhs >= 0 && rhs >= 0;
    }
    bool is_iota(int v, int64_t axis) const {
        const Instr* p = producer(strip(v));
        return p && p->op == OpKind::Iota && p->axis == axis;
    }
    // packed-QKV column block: Reshape(dims)(Slice(qkv,[0,col],[T,width])), optionally transposed
    bool m_qkv_block(int v, bool transposed, int& qkv, int64_t& col, int64_t& width) const {
        v = strip(v);
        if (transposed) { int t; if (!transpose102(v, t)) return false; v = strip(t); }
        int sl;
        if (!reshape_of(v, sl)) return false;
        std::vector<int64_t> s, z;
        if (!slice(strip(sl), qkv, s, z) || s.size() != 2 || s[0] != 0) return false;
        col = s[1];
        width = z[1];
        return true;
    }

    static bool decode_kernel_ok(DType dt, int64_t hq, int64_t hkv, int64_t dh) {
        const int64_t vec = 16 / (int64_t)dtype_size(dt);
        if (dh % vec || dh > 256) return false;
        const int64_t lpr = dh / vec;
        if (lpr > 64 || (lpr & (lpr - 1))) return false;
        const int64_t g = hq / hkv;
        return g == 1 || g == 2 || g == 4 || g == 8;
    }

    void pass_attention() {
        for (size_t i = 0; i < fn.body.size(); ++i) {
            Instr& in = fn.body[i];
            if (in.dead || in.op != OpKind::Reshape) continue;
            const Spec out = in.out_specs[0];
            if (out.rank() != 2 || !dtype_is_float(out.dtype) || in.operands[0].value < 0) continue;
            const int64_t T = out.dims[0];
            int c = strip(in.operands[0].value);
            bool prefill = false;
            { int t; if (transpose102(c, t)) { prefill = true; c = strip(t); } }
            int P, Vg;
            if (!is_dot(c, {0}, {0}, {2}, {1}, P, Vg)) continue;
            const Spec* cs = spec_of(c);
            if (!cs || cs->rank() != 3 || cs->dims[1] != T) continue;
            const int64_t hq = cs->dims[0], dh = cs->dims[2];
            if (out.dims[1] != hq * dh) continue;
            const Instr* sm = producer(strip(P));
            if (!sm || sm->op != OpKind::FSoftmax) continue;
            const int S3 = sm->operands[0].value;
            const Spec* ss = spec_of(S3);
            if (!ss || ss->rank() != 3) continue;
            const int64_t L = ss->dims[2];  // keys attended (capacity in decode, T in prefill)
            int S2, mk, S, scb, Q, Kg;
            float scale;
            auto is_mask = [&](int q) { const Instr* p = producer(strip(q)); return p && p->op == OpKind::BroadcastTo; };
            if (!binary_comm(S3, BinaryOp::Add, S2, mk, is_mask)) continue;
            if (!binary(S2, BinaryOp::Mul, S, scb) || !scalar(scb, scale)) continue;
            if (!is_dot(S, {0}, {0}, {2}, {2}, Q, Kg)) continue;
            int Ksrc, Vsrc;
            int64_t hkv, hkv2;
            if (!group_source(Kg, hq, L, dh, Ksrc, hkv) || !group_source(Vg, hq, L, dh, Vsrc, hkv2) || hkv != hkv2) continue;
            // mask: BroadcastTo chain down to the Select
            int mv = mk;
            for (int d = 0; d < 3; ++d) { int src; if (bcast(mv, src)) mv = src; else break; }
            // a growing cache: the rows of the mask plane that belong to the new tokens, Slice([C, 0], [T, L])
            int64_t mask_row0 = 0;
            {
                int msrc;
                std::vector<int64_t> ms, mz;
                if (slice(strip(mv), msrc, ms, mz) && ms.size() == 2 && ms[1] == 0 && mz[0] == T && mz[1] == L) { mask_row0 = ms[0]; mv = msrc; }
            }
            int cl, cr;
            if (!m_mask_select(mv, cl, cr)) continue;
            int qkv, qkv2, qkv3;
            int64_t col, width;
            if (!prefill) {
                if (T != 1) continue;
                // K' = DynamicUpdateSlice(cacheK, Reshape(Slice(qkv)), update_starts), same for V'
                const Instr* ku = producer(strip(Ksrc));
                const Instr* vu = producer(strip(Vsrc));
                if (!ku || !vu || ku->op != OpKind::DynamicUpdateSlice || vu->op != OpKind::DynamicUpdateSlice) continue;
                if (ku->operands[2].value < 0 || ku->operands[2].value != vu->operands[2].value) continue;
                if (ku->a != std::vector<int64_t>{hkv, 1, dh} || vu->a != ku->a) continue;
                const int cache_k = ku->operands[0].value, cache_v = vu->operands[0].value;
                if (cache_k < 0 || cache_v < 0 || ku->operands[1].value < 0 || vu->operands[1].value < 0) continue;
                if (!m_qkv_block(Q, false, qkv, col, width) || col != 0 || width != hq * dh) continue;
                if (!m_qkv_block(ku->operands[1].value, false, qkv2, col, width) || qkv2 != qkv || col != hq * dh || width != hkv * dh) continue;
                if (!m_qkv_block(vu->operands[1].value, false, qkv3, col, width) || qkv3 != qkv || col != (hq + hkv) * dh || width != hkv * dh) continue;
                const Spec* qs = spec_of(qkv);
                if (!qs || qs->dims != std::vector<int64_t>{1, (hq + 2 * hkv) * dh}) continue;
                // mask compare: BroadcastTo([C])(DynamicSlice{[1]}(iota, query_start)) >= iota
                int qp, ds_src;
                if (!is_iota(cr, 0) || !bcast(cl, qp)) continue;
                const Instr* dsl = producer(strip(qp));
                if (!dsl || dsl->op != OpKind::DynamicSlice || dsl->a != std::vector<int64_t>{1}) continue;
                ds_src = dsl->operands[0].value;
                if (ds_src < 0 || !is_iota(ds_src, 0) || dsl->operands[1].value < 0) continue;
                const Spec* ios = spec_of(strip(ds_src));
                if (!ios || ios->dims != std::vector<int64_t>{L}) continue;
                if (!decode_kernel_ok(out.dtype, hq, hkv, dh)) continue;
                const int kout = ku->out_ids[0], vout = vu->out_ids[0];
                Instr ni = make(OpKind::FAttnDecode, "fused.attention_decode_cache",
                                {qkv, cache_k, cache_v, ku->operands[2].value, dsl->operands[1].value}, in.out_ids[0], out);
                ni.out_ids = {in.out_ids[0], kout, vout};
                ni.out_specs = {out, ku->out_specs[0], vu->out_specs[0]};
                ni.n_q = hq; ni.n_kv = hkv; ni.head_dim = dh; ni.scale = scale;
                kill(kout);
                kill(vout);
                replace_root(in.out_ids[0], ni);
                reindex();
            } else if (L > T) {
                // attention over a growing cache (attention.rs:359-437): K = Concat_1(cache_k, new K rows), same for V,
                // causal mask rows C .. C + T - 1 of the [L, L] plane
                const int64_t C = L - T;
                if (mask_row0 != C || dh > 256 || hq % hkv) continue;
                if (!is_iota(cl, 0) || !is_iota(cr, 1)) continue;
                const Spec* i0 = spec_of(strip(cl));
                if (!i0 || i0->dims != std::vector<int64_t>{L, L}) continue;
                const Instr* kc = producer(strip(Ksrc));
                const Instr* vc = producer(strip(Vsrc));
                if (!kc || !vc || kc->op != OpKind::Concat || vc->op != OpKind::Concat || kc->axis != 1 || vc->axis != 1) continue;
                if (kc->operands.size() != 2 || vc->operands.size() != 2) continue;
                const int cache_k = kc->operands[0].value, cache_v = vc->operands[0].value;
                if (cache_k < 0 || cache_v < 0 || kc->operands[1].value < 0 || vc->operands[1].value < 0) continue;
                const Spec* cks = spec_of(cache_k);
                const Spec* cvs = spec_of(cache_v);
                if (!cks || !cvs || cks->dims != std::vector<int64_t>{hkv, C, dh} || cvs->dims != cks->dims) continue;
                if (cks->dtype != out.dtype || cvs->dtype != out.dtype) continue;
                if (!m_qkv_block(Q, true, qkv, col, width) || col != 0 || width != hq * dh) continue;
                if (!m_qkv_block(kc->operands[1].value, true, qkv2, col, width) || qkv2 != qkv || col != hq * dh || width != hkv * dh) continue;
                if (!m_qkv_block(vc->operands[1].value, true, qkv3, col, width) || qkv3 != qkv || col != (hq + hkv) * dh || width != hkv * dh) continue;
                const Spec* qs = spec_of(qkv);
                if (!qs || qs->dims != std::vector<int64_t>{T, (hq + 2 * hkv) * dh}) continue;
                const int kout = kc->out_ids[0], vout = vc->out_ids[0];
                Instr ni = make(OpKind::FAttnConcat, "fused.attention_concat_cache", {qkv, cache_k, cache_v}, in.out_ids[0], out);
                ni.out_ids = {in.out_ids[0], kout, vout};
                ni.out_specs = {out, kc->out_specs[0], vc->out_specs[0]};
                ni.n_q = hq; ni.n_kv = hkv; ni.head_dim = dh; ni.scale = scale;
                kill(kout);
                kill(vout);
                replace_root(in.out_ids[0], ni);
                reindex();
            } else {
                if (L != T || dh > 256 || mask_row0 != 0) continue;
                if (!is_iota(cl, 0) || !is_iota(cr, 1)) continue;
                const Spec* i0 = spec_of(strip(cl));
                if (!i0 || i0->dims != std::vector<int64_t>{T, T}) continue;
                if (!m_qkv_block(Q, true, qkv, col, width) || col != 0 || width != hq * dh) continue;
                if (!m_qkv_block(Ksrc, true, qkv2, col, width) || qkv2 != qkv || col != hq * dh || width != hkv * dh) continue;
                if (!m_qkv_block(Vsrc, true, qkv3, col, width) || qkv3 != qkv || col != (hq + hkv) * dh || width != hkv * dh) continue;
                const Spec* qs = spec_of(qkv);
                if (!qs || qs->dims != std::vector<int64_t>{T, (hq + 2 * hkv) * dh}) continue;
                if (hq % hkv) continue;
                Instr ni = make(OpKind::FAttnPrefill, "fused.attention_prefill", {qkv}, in.out_ids[0], out);
                ni.n_q = hq; ni.n_kv = hkv; ni.head_dim = dh; ni.scale = scale;
                replace_root(in.out_ids[0], ni);
            }
        }
    }

    // Decode attention reads Q and the new K row straight from the projection; a packed-QKV RoPE
    // that feeds only that attention is applied on load (and to the appended cache row) instead
    // of in a kernel of its own.
    void pass_rope_into_attention() {
        const std::vector<int> uses = count_uses();
        for (auto& at : fn.body) {
            if (at.dead || at.op != OpKind::FAttnDecode || at.rot_half > 0) continue;
            const int qv = at.operands[0].value;
            if (qv < 0 || def[qv] < 0 || uses[qv] != 1) continue;
            Instr& rp = fn.body[def[qv]];
            if (rp.op != OpKind::FRope || rp.dead) continue;
            const int64_t vec = 16 / (int64_t)dtype_size(at.out_specs[0].dtype);
            if (rp.rot_half % vec || rp.head_dim != at.head_dim || rp.n_q != at.n_q || rp.n_kv != at.n_kv) continue;
            at.operands[0] = rp.operands[0];
            at.operands.push_back(rp.operands[1]);
            at.operands.push_back(rp.operands[2]);
            at.rot_half = rp.rot_half;
            rp.dead = true;
            ++fused;
        }
        reindex();
    }

    // Batched decode (the reference has no batch dimension: a batch is B independent sequences whose rows share the
    // linear layers): Concat_0(ctx_0 .. ctx_{B-1}) of B decode attentions over the rows Slice([b,0],[1,P]) of one
    // stacked projection, with the same position operands, becomes ONE attention over all sequences.
    void pass_attention_batch() {
        const std::vector<int> uses = count_uses();
        for (size_t ci = 0; ci < fn.body.size(); ++ci) {
            Instr& cc = fn.body[ci];
            if (cc.dead || cc.op != OpKind::Concat || cc.axis != 0) continue;
            const int64_t B = (int64_t)cc.operands.size();
            if (B < 2 || B > 16) continue;
            std::vector<Instr*> ats, sls;
            int src = -1;
            bool ok = true;
            for (int64_t b = 0; b < B && ok; ++b) {
                const int cv = cc.operands[b].value;
                ok = cv >= 0 && def[cv] >= 0 && uses[cv] == 1;
                if (!ok) break;
                Instr* at = &fn.body[def[cv]];
                ok = at->op == OpKind::FAttnDecode && !at->dead && at->batch <= 1 && at->out_ids[0] == cv;
                if (!ok) break;
                const int qv = at->operands[0].value;
                ok = qv >= 0 && def[qv] >= 0 && uses[qv] == 1;
                if (!ok) break;
                Instr* sl = &fn.body[def[qv]];
                const Spec* ss = sl->op == OpKind::Slice && !sl->dead ? spec_of(sl->operands[0].value) : nullptr;
                ok = ss && ss->rank() == 2 && ss->dims[0] == B && sl->a == std::vector<int64_t>{b, 0} &&
                     sl->b == std::vector<int64_t>{1, ss->dims[1]};
                if (!ok) break;
                if (b == 0) src = sl->operands[0].value;
                ok = sl->operands[0].value == src;
                if (ok && b > 0) {
                    const Instr* a0 = ats[0];
                    ok = at->n_q == a0->n_q && at->n_kv == a0->n_kv && at->head_dim == a0->head_dim && at->rot_half == a0->rot_half &&
                         at->scale == a0->scale && at->operands.size() == a0->operands.size() && at->out_specs == a0->out_specs;
                    for (size_t o = 3; o < at->operands.size() && ok; ++o) ok = at->operands[o].value >= 0 && at->operands[o].value == a0->operands[o].value;
                    const Spec* k0 = spec_of(a0->operands[1].value);
                    const Spec* kb = spec_of(at->operands[1].value);
                    ok = ok && k0 && kb && *k0 == *kb;
                }
                ats.push_back(at);
                sls.push_back(sl);
            }
            if (!ok || (int64_t)ats.size() != B) continue;
            Instr ni = *ats[0];
            ni.batch = B;
            ni.operands[0] = sls[0]->operands[0];
            for (int64_t b = 1; b < B; ++b) {
                ni.operands.push_back(ats[b]->operands[1]);
                ni.operands.push_back(ats[b]->operands[2]);
            }
            ni.out_ids = {cc.out_ids[0]};
            ni.out_specs = {cc.out_specs[0]};
            for (int64_t b = 0; b < B; ++b) {
                ni.out_ids.push_back(ats[b]->out_ids[1]); ni.out_specs.push_back(ats[b]->out_specs[1]);
                ni.out_ids.push_back(ats[b]->out_ids[2]); ni.out_specs.push_back(ats[b]->out_specs[2]);
            }
            ni.op_name = "fused.attention_decode_batch";
            for (Instr* a : ats) a->dead = true;
            for (Instr* sl : sls) sl->dead = true;
            fn.body[ci] = ni;
            ++fused;
            reindex();
        }
    }

    // ---------------------------------------------------------------- linear layers
    std::vector<int> count_uses() const {
        std::vector<int> uses(fn.max_value_id + 1, 0);
        for (auto& in : fn.body)
            if (!in.dead)
                for (auto& o : in.operands)
                    if (o.value >= 0) ++uses[o.value];
        for (int r : fn.result_ids) ++uses[r];
        return uses;
    }

    // 0: the generic kernels; 1: matrix-core GEMM over a k-grouped copy; 2: weight-streaming decode kernels over a
    // tiled copy (the persistent chain, the batched matrix-core kernel, the tiled GEMV).  Needs weights (and scales)
    // that are program inputs.  Works on a Dot as well as on an FLinear (operand 0 = x, 1 = W).
    int linear_path(const Instr& in) const {
        auto is_param = [&](int v) { return v >= 0 && def[v] < 0 && spec_of(v) != nullptr; };
        const Spec* xs = spec_of(in.operands[0].value);
        const Spec* ws = spec_of(in.operands[1].value);
        if (!xs || !ws || xs->rank() != 2 || ws->rank() != 2) return 0;
        const int64_t M = xs->dims[0], K = xs->dims[1], N = ws->dims[1];
        // with a folded f32 norm x is f32 while the kernel computes in the weights' dtype
        const int dt = in.quant ? (int)spec_of(in.operands[2].value)->dtype : (int)ws->dtype;
        if (!is_param(in.operands[1].value)) return 0;
        if (in.act == 2 && !is_param(in.operands[linear_w2_pos(in)].value)) return 0;
        if (in.quant && (!is_param(in.operands[2].value) || (in.act == 2 && !is_param(in.operands[4].value)))) return 0;
        if (k::mfma_gemm_supported(dt, M, K, N, in.quant)) return 1;
        if (in.quant)   // decode: the persistent chain (one row) and the batched matrix-core kernel read the codes directly
            return (k::chain_supported(dt, M, K, N, in.act == 2, false, in.quant) || k::skinny_quant_supported(dt, M, K, N, in.quant)) ? 2 : 0;
        if (!k::gemv_tiled_supported(dt, M, K, N)) return 0;
        // SwiGLU pairs: the vector kernel holds up to 8 rows, the matrix-core kernel of batched decode up to 16
        if (in.act == 2 && M > 8 && !k::skinny_gemm_supported(dt, M, K, N)) return 0;
        return 2;
    }
    bool fast_linear(const Instr& in) const { return linear_path(in) != 0; }

    void pass_linear() {
        // 1. x[M,K] . W[K,N] -> FLinear
        for (auto& in : fn.body) {
            if (in.dead || in.op != OpKind::Dot) continue;
            if (!in.a.empty() || !in.b.empty() || in.c != std::vector<int64_t>{1} || in.d != std::vector<int64_t>{0}) continue;
            if (in.operands[0].value < 0 || in.operands[1].value < 0) continue;
            const Spec* l = spec_of(in.operands[0].value);
            const Spec* r = spec_of(in.operands[1].value);
            if (!l || !r || l->rank() != 2 || r->rank() != 2 || !dtype_is_float(l->dtype)) continue;
            // an f32 result over bf16 operands is stored by the weight-streaming and matrix-core kernels only
            if (in.out_f32 && !fast_linear(in)) continue;
            in.op = OpKind::FLinear;
            in.op_name = "fused.linear";
            in.act = 0;
            ++fused;
        }
        // quantised dots (already validated as written) take the same epilogues
        for (auto& in : fn.body) {
            if (in.dead || in.op != OpKind::CustomCall) continue;
            const int q = quant_dot_target(in.target);
            if (!q || in.operands.size() != 3) continue;
            bool vals = true;
            for (auto& o : in.operands) vals = vals && o.value >= 0;
            if (!vals) continue;
            in.op = OpKind::FLinear;
            in.op_name = q == 1 ? "fused.linear_w8" : "fused.linear_w4g128";
            in.quant = q;
            in.act = 0;
            const Spec* xs = spec_of(in.operands[0].value);   // the accumulator leaves as f32 when the call's output is declared so
            in.out_f32 = xs && xs->dtype == DType::BF16 && in.out_specs[0].dtype == DType::F32;
        }
        reindex();
        // 2. epilogues, each absorbed only when the linear's value has no other reader
        bool changed = true;
        while (changed) {
            changed = false;
            const std::vector<int> uses = count_uses();
            for (size_t i = 0; i < fn.body.size() && !changed; ++i) {
                Instr& in = fn.body[i];
                if (in.dead) continue;
                const int v = in.out_ids[0];
                auto linear_of = [&](int q) -> Instr* {
                    if (q < 0 || def[q] < 0) return nullptr;
                    Instr* p = &fn.body[def[q]];
                    return (p->op == OpKind::FLinear && !p->dead && uses[q] == 1) ? p : nullptr;
                };
                if (in.op == OpKind::Binary && in.binary == BinaryOp::Add && !in.scalar_rhs) {
                    const int a = in.operands[0].value, b = in.operands[1].value;
                    if (a < 0 || b < 0) continue;
                    // bias: Add(linear, BroadcastTo(b[N]))  (tensor_ops.rs:42-56)
                    Instr* lin = linear_of(a);
                    int vec;
                    if (lin && !lin->has_bias && !lin->has_residual && lin->act == 0 && !lin->out_f32 &&
                        vector_bcast_last(b, in.out_specs[0].dims.back(), vec)) {
                        Instr ni = *lin;
                        Operand o; o.value = vec;
                        ni.operands.push_back(o);
                        ni.has_bias = true;
                        ni.out_ids = {v};
                        lin->dead = true;
                        fn.body[i] = ni;
                        reindex();
                        changed = true;
                        continue;
                    }
                    // residual: Add(linear, r) or Add(r, linear)
                    for (int side = 0; side < 2 && !changed; ++side) {
                        Instr* l2 = linear_of(side == 0 ? a : b);
                        const int other = side == 0 ? b : a;
                        if (!l2 || l2->has_residual || l2->act == 2) continue;
                        if (l2->out_f32 && !fast_linear(*l2)) continue;   // (a quantised linear outside the fast kernels)
                        if (def[other] >= 0 && def[other] > def[l2->out_ids[0]]) {
                            // the residual is produced after the linear: fine, the fused op sits at the Add
                        }
                        const Spec* os = spec_of(other);
                        if (!os || *os != in.out_specs[0]) continue;
                        Instr ni = *l2;
                        Operand o; o.value = other;
                        ni.operands.push_back(o);
                        ni.has_residual = true;
                        ni.out_ids = {v};
                        l2->dead = true;
                        fn.body[i] = ni;
                        reindex();
                        changed = true;
                    }
                } else if (in.op == OpKind::FGelu) {
                    Instr* lin = linear_of(in.operands[0].value);
                    if (lin && lin->act == 0 && !lin->has_residual && !lin->out_f32 && in.fparam[0] == 0.5f && in.fparam[1] == 1.41421354f &&
                        in.fparam[2] == 1.0f) {
                        Instr ni = *lin;
                        ni.act = 1;
                        ni.out_ids = {v};
                        lin->dead = true;
                        fn.body[i] = ni;
                        reindex();
                        changed = true;
                    }
                } else if (in.op == OpKind::FSwiglu) {
                    Instr* lg = linear_of(in.operands[0].value);
                    Instr* lu = linear_of(in.operands[1].value);
                    if (lg && lu && lg != lu && lg->act == 0 && lu->act == 0 && !lg->has_bias && !lu->has_bias &&
                        !lg->out_f32 && !lu->out_f32 &&
                        !lg->has_residual && !lu->has_residual && lg->operands[0].value == lu->operands[0].value &&
                        lg->quant == lu->quant) {
                        const Spec* wg = spec_of(lg->operands[1].value);
                        const Spec* wu = spec_of(lu->operands[1].value);
                        if (wg && wu && *wg == *wu) {
                            Instr ni = *lg;
                            ni.operands.push_back(lu->operands[1]);
                            if (lg->quant) ni.operands.push_back(lu->operands[2]);
                            ni.act = 2;
                            ni.out_ids = {v};
                            lg->dead = true;
                            lu->dead = true;
                            fn.body[i] = ni;
                            reindex();
                            changed = true;
                        }
                    }
                }
            }
        }
    }

    // Decode-sized linears whose weights are program inputs run over the column-tiled weight copy;
    // an RMSNorm feeding only such linears is folded into them (every block reads the whole row of x
    // anyway, so the row statistic is free).
    void pass_tiled_linear() {
        for (auto& in : fn.body) {
            if (in.dead || in.op != OpKind::FLinear) continue;
            const int path = linear_path(in);
            in.mfma = path == 1;
            in.tiled = path == 2;
        }
        const std::vector<int> uses = count_uses();
        std::vector<bool> is_result(fn.max_value_id + 1, false);
        for (int r : fn.result_ids) is_result[r] = true;
        for (size_t i = 0; i < fn.body.size(); ++i) {
            Instr& nrm = fn.body[i];
            if (nrm.dead || (nrm.op != OpKind::FRmsNorm && nrm.op != OpKind::FLayerNorm)) continue;
            const bool ln = nrm.op == OpKind::FLayerNorm;   // folded into plain (unquantised) decode linears only
            const int nv = nrm.out_ids[0];
            if (is_result[nv] || nrm.out_specs[0].rank() != 2) continue;
            const Spec* nx = spec_of(nrm.operands[0].value);
            const bool xf32 = nx && nx->dtype == DType::F32 && nrm.out_specs[0].dtype == DType::BF16;
            std::vector<Instr*> cons;
            int found = 0;
            for (auto& c : fn.body) {
                if (c.dead) continue;
                for (size_t o = 0; o < c.operands.size(); ++o) {
                    if (c.operands[o].value != nv) continue;
                    ++found;
                    if (c.op == OpKind::FLinear && c.tiled && !c.norm && o == 0 && !(ln && c.quant) && !(ln && xf32)) cons.push_back(&c);
                }
            }
            if (cons.empty() || (int)cons.size() != found || found != uses[nv]) continue;
            for (Instr* c : cons) {
                c->operands[0] = nrm.operands[0];
                c->operands.push_back(nrm.operands[1]);
                if (ln) c->operands.push_back(nrm.operands[2]);
                c->norm = true;
                c->x_f32 = xf32;
                c->norm_ln = ln;
                c->eps = nrm.eps;
                c->scale = nrm.scale;
            }
            nrm.dead = true;
            ++fused;
        }
        reindex();
    }

    // Binary ops whose rhs is a broadcast scalar literal read the scalar as a kernel argument.
    void pass_scalar_rhs() {
        for (auto& in : fn.body) {
            if (in.dead || in.op != OpKind::Binary || in.scalar_rhs) continue;
            const int b = in.operands[1].value;
            float val;
            if (b < 0 || !scalar(b, val)) continue;
            const Instr* p = producer(b);
            if (!p || p->op != OpKind::BroadcastTo) continue;
            in.scalar_rhs = true;
            in.scalar_val = val;
            in.operands.resize(1);
        }
    }

    // DynamicUpdateSlice(base, view(x), starts), where view is a chain of Slice / Reshape / Transpose instructions
    // that nothing else reads, copies straight out of x: the chain only renumbers elements, so its composition is a
    // set of strides and an offset inside x.  (A prefill writes the K and V rows of the packed projection into the
    // caches this way: four copies per layer become none.)
    static bool reshape_view(const std::vector<int64_t>& od, const std::vector<int64_t>& os, const std::vector<int64_t>& nd,
                             std::vector<int64_t>& ns) {
        // strides of the new shape over the same elements, if the old view allows it without a copy
        ns.assign(nd.size(), 0);
        size_t oi = 0, ni = 0;
        while (oi < od.size() && ni < nd.size()) {
            // grow a group of old axes and a group of new axes until they hold the same number of elements
            size_t oj = oi + 1, nj = ni + 1;
            int64_t op = od[oi], np = nd[ni];
            while (op != np) {
                if (op < np) { if (oj >= od.size()) return false; op *= od[oj++]; }
                else { if (nj >= nd.size()) return false; np *= nd[nj++]; }
            }
            // the old group must be contiguous in itself (axes of extent 1 carry no constraint)
            for (size_t k = oi; k + 1 < oj; ++k)
                if (od[k] != 1 && od[k + 1] != 1 && os[k] != os[k + 1] * od[k + 1]) return false;
            int64_t inner = 1;
            for (size_t k = oj; k-- > oi;) if (od[k] != 1) { inner = os[k]; break; }
            for (size_t k = nj; k-- > ni;) { ns[k] = inner; inner *= nd[k]; }
            oi = oj; ni = nj;
        }
        for (; oi < od.size(); ++oi) if (od[oi] != 1) return false;
        for (; ni < nd.size(); ++ni) { if (nd[ni] != 1) return false; ns[ni] = 1; }
        return true;
    }
    void pass_update_views() {
        const std::vector<int> uses = count_uses();
        for (auto& in : fn.body) {
            if (in.dead || in.op != OpKind::DynamicUpdateSlice || !in.view_dims.empty()) continue;
            // the chain, from the update up to its root
            std::vector<const Instr*> chain;
            int v = in.operands[1].value;
            for (;;) {
                const Instr* p = producer(v);
                if (!p || uses[v] != 1 || p->operands.empty() || p->operands[0].value < 0) break;
                if (p->op != OpKind::Slice && p->op != OpKind::Reshape && p->op != OpKind::Transpose) break;
                chain.push_back(p);
                v = p->operands[0].value;
            }
            bool copies = false;
            for (const Instr* p : chain) copies = copies || p->op != OpKind::Reshape;
            if (!copies) continue;   // reshapes alone cost nothing
            // a view of the base itself must be taken before the base is written (the update may run in place)
            auto storage = [&](int x) {
                for (const Instr* p = producer(x); p && p->op == OpKind::Reshape && p->operands[0].value >= 0; p = producer(x))
                    x = p->operands[0].value;
                return x;
            };
            if (storage(v) == storage(in.operands[0].value)) continue;
            const Spec* root = spec_of(v);
            if (!root || root->rank() > k::kMaxRank) continue;
            std::vector<int64_t> dims = root->dims, strides(root->rank(), 1);
            for (int i = root->rank() - 2; i >= 0; --i) strides[i] = strides[i + 1] * dims[i + 1];
            int64_t off = 0;
            bool ok = true;
            for (size_t c = chain.size(); ok && c-- > 0;) {
                const Instr* p = chain[c];
                if (p->op == OpKind::Slice) {
                    for (size_t i = 0; i < dims.size(); ++i) off += p->a[i] * strides[i];
                    dims = p->b;
                } else if (p->op == OpKind::Transpose) {
                    std::vector<int64_t> d2(dims.size()), s2(dims.size());
                    for (size_t i = 0; i < dims.size(); ++i) { d2[i] = dims[p->a[i]]; s2[i] = strides[p->a[i]]; }
                    dims = d2; strides = s2;
                } else {
                    std::vector<int64_t> s2;
                    ok = reshape_view(dims, strides, p->out_specs[0].dims, s2);
                    dims = p->out_specs[0].dims; strides = s2;
                }
                ok = ok && (int)dims.size() <= k::kMaxRank;
            }
            const Spec* upd = spec_of(in.operands[1].value);
            if (!ok || !upd || dims != upd->dims) continue;
            in.view_dims = dims;
            in.view_strides = strides;
            in.view_off = off;
            in.operands[1].value = v;
            ++fused;
        }
    }

    void dce() {
        std::vector<bool> live(fn.max_value_id + 1, false);
        for (int r : fn.result_ids) live[r] = true;
        for (int i = (int)fn.body.size() - 1; i >= 0; --i) {
            Instr& in = fn.body[i];
            if (in.dead) continue;
            bool any = false;
            for (int id : in.out_ids) any = any || live[id];
            if (!any) { in.dead = true; continue; }
            for (auto& o : in.operands)
                if (o.value >= 0) live[o.value] = true;
        }
        reindex();
    }

    // Stable topological order: a fused instruction sits at its root's position, which can be
    // before the producer of an operand that the original sequence only read later.
    void toposort() {
        const size_t n = fn.body.size();
        std::vector<bool> placed_val(fn.max_value_id + 1, false);
        for (int p : fn.param_ids) placed_val[p] = true;
        std::vector<bool> done(n, false);
        std::vector<Instr> order;
        order.reserve(n);
        size_t remaining = 0;
        for (auto& in : fn.body) if (!in.dead) ++remaining;
        while (remaining) {
            bool progress = false;
            for (size_t i = 0; i < n; ++i) {
                if (done[i] || fn.body[i].dead) continue;
                bool ready = true;
                for (auto& o : fn.body[i].operands)
                    if (o.value >= 0 && !placed_val[o.value]) { ready = false; break; }
                if (!ready) continue;
                for (int id : fn.body[i].out_ids) placed_val[id] = true;
                order.push_back(fn.body[i]);
                done[i] = true;
                --remaining;
                progress = true;
            }
            if (!progress) fail_exec("operand value missing");
        }
        fn.body = std::move(order);
        reindex();
    }
};

}  // namespace

void lower_norm_calls(Function& fn) {
    auto spec_of = [&](int v) -> const Spec* {
        for (size_t i = 0; i < fn.param_ids.size(); ++i)
            if (fn.param_ids[i] == v) return &fn.param_specs[i];
        for (const Instr& in : fn.body)
            for (size_t o = 0; o < in.out_ids.size(); ++o)
                if (in.out_ids[o] == v) return &in.out_specs[o];
        return nullptr;
    };
    for (Instr& in : fn.body) {
        if (in.op != OpKind::CustomCall) continue;
        const int kind = norm_call_target(in.target);
        if (!kind) continue;
        const size_t want = kind == 1 ? 3 : 2;
        if (in.operands.size() != want) fail_spec(in.target + ": expects " + std::string(kind == 1 ? "(x, gamma, beta)" : "(x, gamma)"));
        const Spec* xs = in.operands[0].value >= 0 ? spec_of(in.operands[0].value) : nullptr;
        if (!xs || !dtype_is_float(xs->dtype) || xs->rank() < 1) fail_spec(in.target + ": x must be a float tensor of rank >= 1");
        const int64_t n = xs->dims.back();
        for (size_t o = 1; o < want; ++o) {
            const Spec* vs = in.operands[o].value >= 0 ? spec_of(in.operands[o].value) : nullptr;
            if (!vs || vs->dtype != xs->dtype || vs->dims != std::vector<int64_t>{n})
                fail_spec(in.target + ": gamma / beta must be [" + std::to_string(n) + "] of x's dtype");
        }
        if (in.out_specs[0] != *xs) fail_spec(in.target + ": the output has x's type");
        auto it = in.attrs.find("eps");
        const Json* val = it == in.attrs.end() ? nullptr : it->second.find("value");
        if (!val) fail_spec(in.target + ": attribute `eps` (F64) is missing");
        try {
            in.eps = (float)val->as_double();
        } catch (const JsonError&) {
            fail_spec(in.target + ": attribute `eps` must be a number");
        }
        if (!(in.eps > 0.0f) || !std::isfinite(in.eps)) fail_spec(in.target + ": eps must be positive and finite");
        in.scale = 1.0f / (float)n;   // the functional's own literal (normalization.rs:123-217: 1.0 / n as f32)
        in.op = kind == 1 ? OpKind::FLayerNorm : OpKind::FRmsNorm;
        in.op_name = kind == 1 ? "fused.layer_norm" : "fused.rms_norm";
    }
}

std::vector<BroadcastInput> expand_broadcast_inputs(Function& fn, const std::vector<const Spec*>& src) {
    std::vector<BroadcastInput> out;
    std::vector<Instr> front;
    const size_t n_in = fn.param_ids.size();
    for (size_t i = 0; i < n_in && i < src.size(); ++i) {
        if (!src[i]) continue;
        const Spec full = fn.param_specs[i];
        const Spec& vec = *src[i];
        if (vec.dtype != full.dtype || vec.rank() < 1 || full.rank() < 1 || vec.rank() > full.rank()) continue;
        if (vec.dims.back() != full.dims.back() || vec.count() != vec.dims.back()) continue;
        BroadcastInput b;
        b.input = (int)i;
        b.param_value = ++fn.max_value_id;
        b.bcast_value = ++fn.max_value_id;
        const int v = fn.param_ids[i];
        bool read = false;
        for (auto& in : fn.body)
            for (auto& o : in.operands)
                if (o.value == v) { o.value = b.bcast_value; read = true; }
        if (!read) { fn.max_value_id -= 2; continue; }
        fn.param_ids.push_back(b.param_value);
        fn.param_specs.push_back(vec);
        Instr bc;
        bc.op = OpKind::BroadcastTo;
        bc.op_name = "BroadcastTo";
        Operand o; o.value = b.param_value;
        bc.operands = {o};
        bc.out_ids = {b.bcast_value};
        bc.out_specs = {full};
        front.push_back(std::move(bc));
        out.push_back(b);
    }
    fn.body.insert(fn.body.begin(), front.begin(), front.end());
    return out;
}

void collapse_broadcast_inputs(Function& fn, const std::vector<BroadcastInput>& expanded) {
    for (const BroadcastInput& b : expanded) {
        const int v = fn.param_ids[b.input];
        for (auto& in : fn.body) {
            if (in.dead) continue;
            if (in.op == OpKind::BroadcastTo && in.out_ids[0] == b.bcast_value) { in.dead = true; continue; }
            for (auto& o : in.operands)
                if (o.value == b.bcast_value) o.value = v;
        }
    }
}

int result_broadcast_source(const Function& fn, size_t r) {
    if (r >= fn.result_ids.size() || fn.result_specs[r].rank() < 1) return -1;
    const int64_t n = fn.result_specs[r].dims.back();
    int v = fn.result_ids[r];
    bool widened = false;
    for (int depth = 0; depth < 8; ++depth) {
        for (size_t i = 0; i < fn.param_ids.size(); ++i)
            if (fn.param_ids[i] == v) {
                const Spec& s = fn.param_specs[i];
                return (widened && s.rank() >= 1 && s.dims.back() == n && s.count() == n) ? (int)i : -1;
            }
        const Instr* p = nullptr;
        for (const Instr& in : fn.body)
            if (!in.dead && in.out_ids[0] == v) { p = &in; break; }
        if (!p || (p->op != OpKind::BroadcastTo && p->op != OpKind::Reshape)) return -1;
        if (p->operands.size() != 1 || p->operands[0].value < 0) return -1;
        if (p->out_specs[0].rank() < 1 || p->out_specs[0].dims.back() != n) return -1;
        widened = widened || p->op == OpKind::BroadcastTo;
        v = p->operands[0].value;
    }
    return -1;
}

int fuse_function(Function& fn) {
    Fuser f(fn);
    f.dce();
    f.pass_split_slices();
    f.pass_elementwise();
    f.dce();
    f.pass_norm_cast();
    f.dce();
    f.pass_rope();
    f.pass_attention();
    f.dce();
    f.pass_rope_into_attention();
    f.dce();
    f.pass_attention_batch();
    f.dce();
    f.pass_linear();
    f.dce();
    f.pass_tiled_linear();
    f.dce();
    f.pass_scalar_rhs();
    f.dce();
    f.pass_update_views();
    f.dce();
    f.toposort();
    return f.fused;
}

}  // namespace gptrs
