// Program -> Plan: validate every instruction against docs/backend.md, decide where each SSA
// value lives (input, donated-in-place, output buffer, workspace slice, constant block) and
// precompute one launch descriptor per instruction.  run_step() issues the launches.
#include <algorithm>
#include <cstring>
#include <functional>

#include "runtime.hpp"

namespace gptrs {

// The weight format of a linear layer inside a decode chain: f32 weights have a format of their own, the others follow
// the quantisation of the layer.
static inline int chain_format(const Instr& in, DType ldt) { return ldt == DType::F32 ? k::kChainW32 : (int)in.quant; }

static constexpr size_t kAlign = 256;
static size_t align_up(size_t n) { return (n + kAlign - 1) / kAlign * kAlign; }

static std::vector<int64_t> row_major_strides(const std::vector<int64_t>& dims) {
    std::vector<int64_t> s(dims.size(), 1);
    for (int i = (int)dims.size() - 2; i >= 0; --i) s[i] = s[i + 1] * dims[i + 1];
    return s;
}

// Build a CopyDesc over `dims` with the given element strides, merging adjacent dims that are
// contiguous on both sides and dropping extent-1 dims.
static k::CopyDesc make_copy(const std::vector<int64_t>& dims, const std::vector<int64_t>& dst_stride,
                             const std::vector<int64_t>& src_stride, int64_t dst_off, int64_t src_off) {
    std::vector<int64_t> d, ds, ss;
    for (size_t i = 0; i < dims.size(); ++i) {
        if (dims[i] == 1) continue;
        if (!d.empty() && ds.back() == dst_stride[i] * dims[i] && ss.back() == src_stride[i] * dims[i]) {
            d.back() *= dims[i];
            ds.back() = dst_stride[i];
            ss.back() = src_stride[i];
        } else {
            d.push_back(dims[i]);
            ds.push_back(dst_stride[i]);
            ss.push_back(src_stride[i]);
        }
    }
    if ((int)d.size() > k::kMaxRank) fail_unimpl("copy", "rank above 6 after collapsing");
    k::CopyDesc c;
    c.rank = (int)d.size();
    c.total = 1;
    for (size_t i = 0; i < d.size(); ++i) {
        c.dims[i] = d[i];
        c.dst_stride[i] = ds[i];
        c.src_stride[i] = ss[i];
        c.total *= d[i];
    }
    for (auto x : dims) if (x == 0) c.total = 0;
    c.dst_off = dst_off;
    c.src_off = src_off;
    return c;
}

// Reinterpret a copy of `es`-byte elements as words `f` times wider when every run allows it.
static bool can_widen(const k::CopyDesc& c, int f) {
    if (c.total == 0 || c.rank == 0) return false;
    const int last = c.rank - 1;
    bool ok = c.dst_stride[last] == 1 && c.src_stride[last] == 1 && c.dims[last] % f == 0 && c.dst_off % f == 0 &&
              c.src_off % f == 0;
    for (int i = 0; i < last && ok; ++i) ok = c.dst_stride[i] % f == 0 && c.src_stride[i] % f == 0;
    for (int i = 0; i < c.dyn_rank && ok; ++i) ok = c.dyn_stride[i] % f == 0;
    return ok;
}
static void apply_widen(k::CopyDesc& c, int f) {
    const int last = c.rank - 1;
    c.dims[last] /= f;
    c.total /= f;
    c.dst_off /= f;
    c.src_off /= f;
    for (int i = 0; i < last; ++i) { c.dst_stride[i] /= f; c.src_stride[i] /= f; }
    for (int i = 0; i < c.dyn_rank; ++i) c.dyn_stride[i] /= f;
}
// Widens every piece of one op to a common word size; returns the element size to launch with.
// (Device buffers are 256-byte aligned, so element offsets decide alignment.)
static int widen_copies(std::vector<k::CopyDesc>& cs, int es) {
    for (int w : {16, 8, 4, 2}) {
        if (w <= es || w % es) continue;
        const int f = w / es;
        bool ok = true;
        for (auto& c : cs) ok = ok && (c.total == 0 || can_widen(c, f));
        if (!ok) continue;
        for (auto& c : cs) if (c.total) apply_widen(c, f);
        return w;
    }
    return es;
}

// The dtype an FLinear computes in: its weights' (a quantised one: its scales').  x has it too unless an f32 norm was
// folded in (Instr::x_f32); the result has it unless the accumulator leaves as f32 (Instr::out_f32).
static inline DType linear_dtype(const Instr& in, const Spec& w, const Spec* scales) {
    return in.quant && scales ? scales->dtype : w.dtype;
}

static int64_t norm_axis(int64_t axis, int rank, const char* op) {
    if (axis < 0) axis += rank;
    if (axis < 0 || axis >= rank) fail_exec(std::string(op) + " axis out of range");
    return axis;
}

namespace {
struct Builder {
    Plan& plan;
    const std::vector<bool>& donated;
    std::vector<int> use_count;      // per root value
    std::vector<int> last_use;       // per root value: last step index that reads it
    std::vector<int> def_step;       // per root value
    std::vector<size_t> lit_offset;  // literal index -> const offset
    std::vector<int> param_pos;      // value id -> input position, -1 when not a function parameter

    Builder(Plan& p, const std::vector<bool>& d) : plan(p), donated(d) {}

    const Spec& spec_of(const Instr& in, size_t i) {
        const Operand& o = in.operands[i];
        if (o.value >= 0) {
            if (o.value >= (int)plan.values.size() || !plan.values[o.value].defined) fail_exec("operand value missing");
            return plan.values[o.value].spec;
        }
        return plan.fn.literals[o.literal].spec;
    }
    int root(int v) const {
        while (plan.values[v].root != v) v = plan.values[v].root;
        return v;
    }
    size_t const_add(const std::vector<uint8_t>& bytes) {
        size_t off = align_up(plan.const_host.size());
        plan.const_host.resize(off + std::max<size_t>(bytes.size(), 1), 0);
        if (!bytes.empty()) memcpy(plan.const_host.data() + off, bytes.data(), bytes.size());
        return off;
    }
    void define(int id, const Spec& s) {
        if (id < 0) fail_exec("negative value id");
        if (id >= (int)plan.values.size()) plan.values.resize(id + 1);
        if (plan.values[id].defined) fail_exec("value id defined twice");
        plan.values[id].spec = s;
        plan.values[id].root = id;
        plan.values[id].defined = true;
    }

    void validate(Instr& in);
    void build();
    void describe(Step& st);
};
}  // namespace

static void expect(bool c, const std::string& msg) {
    if (!c) fail_exec(msg);
}

// Shape/dtype rules per op (docs/backend.md "Operation reference"; messages follow cpu.rs).
void Builder::validate(Instr& in) {
    const Spec& out = in.out_specs[0];
    auto same_shape = [&](size_t a, size_t b, const char* what) {
        expect(spec_of(in, a).dims == spec_of(in, b).dims, std::string(what) + " size mismatch");
    };
    switch (in.op) {
        case OpKind::Constant:
            expect(plan.fn.literals[in.literal].spec == out, "constant output spec mismatch");
            break;
        case OpKind::Unary: {
            const Spec& x = spec_of(in, 0);
            expect(dtype_is_float(x.dtype), "elementwise unary only supports f32/bf16 tensors");
            expect(x == out, "elementwise unary output spec mismatch");
            break;
        }
        case OpKind::Binary: {
            const Spec& a = spec_of(in, 0);
            if (in.scalar_rhs) {  // rhs folded to a kernel argument by the fusion pass
                expect(dtype_is_float(a.dtype) && a == out, "elementwise binary output spec mismatch");
                break;
            }
            const Spec& b = spec_of(in, 1);
            expect(a.dtype == b.dtype && dtype_is_float(a.dtype), "elementwise binary only supports f32/bf16 tensors of one dtype");
            same_shape(0, 1, "elementwise");
            expect(a == out, "elementwise binary output spec mismatch");
            break;
        }
        case OpKind::Compare: {
            const Spec& a = spec_of(in, 0);
            const Spec& b = spec_of(in, 1);
            expect(a.dtype == b.dtype && (a.dtype == DType::SI32 || dtype_is_float(a.dtype)), "compare supports si32/f32/bf16 tensors");
            same_shape(0, 1, "compare");
            expect(out.dtype == DType::I1 && out.dims == a.dims, "compare output must be i1 of the operand shape");
            break;
        }
        case OpKind::Select: {
            const Spec& p = spec_of(in, 0);
            const Spec& t = spec_of(in, 1);
            const Spec& f = spec_of(in, 2);
            expect(p.dtype == DType::I1 && t.dtype == f.dtype, "select dtype combination unsupported");
            expect(p.dims == t.dims && t.dims == f.dims && t == out, "select shape mismatch");
            break;
        }
        case OpKind::Cast:
            expect(spec_of(in, 0).dims == out.dims, "cast shape mismatch");
            break;
        case OpKind::StopGradient:
            expect(spec_of(in, 0) == out, "stop_gradient output spec mismatch");
            break;
        case OpKind::Reshape: {
            const Spec& x = spec_of(in, 0);
            expect(x.dtype == out.dtype && x.count() == out.count(), "reshape element count mismatch");
            break;
        }
        case OpKind::Transpose: {
            const Spec& x = spec_of(in, 0);
            expect((int)in.a.size() == x.rank() && x.dtype == out.dtype && out.rank() == x.rank(), "transpose perm rank mismatch");
            std::vector<bool> seen(x.rank(), false);
            for (int i = 0; i < x.rank(); ++i) {
                const int64_t p = in.a[i];
                expect(p >= 0 && p < x.rank() && !seen[p], "transpose perm is not a permutation");
                seen[p] = true;
                expect(out.dims[i] == x.dims[p], "transpose output shape mismatch");
            }
            break;
        }
        case OpKind::BroadcastTo: {
            const Spec& x = spec_of(in, 0);
            expect(x.dtype == out.dtype, "broadcast_to dtype mismatch");
            if (x.rank() > out.rank()) fail_spec("broadcast_to: input rank exceeds result rank");
            const int pad = out.rank() - x.rank();
            for (int i = 0; i < x.rank(); ++i)
                if (x.dims[i] != out.dims[pad + i] && x.dims[i] != 1)
                    fail_spec("broadcast_to: shapes " + x.str() + " and " + out.str() + " are not broadcast-compatible");
            break;
        }
        case OpKind::Slice: {
            const Spec& x = spec_of(in, 0);
            expect((int)in.a.size() == x.rank() && (int)in.b.size() == x.rank(), "slice starts/sizes must match rank");
            for (int i = 0; i < x.rank(); ++i) expect(in.a[i] >= 0 && in.b[i] >= 0 && in.a[i] + in.b[i] <= x.dims[i], "slice exceeds bounds");
            expect(out.dtype == x.dtype && out.dims == in.b, "slice output shape mismatch");
            break;
        }
        case OpKind::Concat: {
            const Spec& x0 = spec_of(in, 0);
            in.axis = norm_axis(in.axis, x0.rank(), "concat");
            int64_t total = 0;
            for (size_t i = 0; i < in.operands.size(); ++i) {
                const Spec& x = spec_of(in, i);
                expect(x.dtype == x0.dtype && x.rank() == x0.rank(), "concat dtype/rank mismatch");
                for (int d = 0; d < x.rank(); ++d)
                    if (d != in.axis) expect(x.dims[d] == x0.dims[d], "concat shape mismatch off the concat axis");
                total += x.dims[in.axis];
            }
            expect(out.dtype == x0.dtype && out.rank() == x0.rank() && out.dims[in.axis] == total, "concat output shape mismatch");
            break;
        }
        case OpKind::Iota:
            expect(out.dtype == DType::SI32, "iota only supports si32");
            expect(in.axis >= 0 && in.axis < out.rank(), "iota axis out of range");
            break;
        case OpKind::Take: {
            const Spec& x = spec_of(in, 0);
            const Spec& idx = spec_of(in, 1);
            expect(x.rank() >= 1, "take requires rank >= 1");
            expect(idx.dtype == DType::SI32, "take indices must be si32");
            std::vector<int64_t> want = idx.dims;
            want.insert(want.end(), x.dims.begin() + 1, x.dims.end());
            expect(out.dtype == x.dtype && out.dims == want, "take output shape mismatch");
            break;
        }
        case OpKind::DynamicSlice: {
            const Spec& x = spec_of(in, 0);
            const Spec& st = spec_of(in, 1);
            expect((int)in.a.size() == x.rank(), "dynamic_slice sizes length must match input rank");
            expect(st.dtype == DType::SI32, "dynamic_slice starts must be si32");
            expect(st.rank() == 1 && st.dims[0] == x.rank(), "dynamic_slice starts must be 1-D of length equal to rank");
            for (int i = 0; i < x.rank(); ++i)
                if (in.a[i] > x.dims[i]) fail_spec("dynamic_slice size exceeds dimension");
            expect(out.dtype == x.dtype && out.dims == in.a, "dynamic_slice output shape mismatch");
            break;
        }
        case OpKind::DynamicUpdateSlice: {
            const Spec& x = spec_of(in, 0);
            const Spec& u = spec_of(in, 1);
            const Spec& st = spec_of(in, 2);
            // after fusion operand 1 may be the tensor the update is a view of (in.view_dims is then the update's shape)
            const std::vector<int64_t>& udims = in.view_dims.empty() ? u.dims : in.view_dims;
            expect(x.dtype == u.dtype, "dynamic_update_slice dtype mismatch");
            expect((int)udims.size() == x.rank() && in.a == udims, "dynamic_update_slice sizes must match update shape");
            expect(st.dtype == DType::SI32 && st.rank() == 1 && st.dims[0] == x.rank(), "dynamic_update_slice starts must be si32[rank]");
            for (int i = 0; i < x.rank(); ++i)
                if (udims[i] > x.dims[i]) fail_spec("dynamic_update_slice update exceeds base dimension");
            expect(out == x, "dynamic_update_slice output spec mismatch");
            break;
        }
        case OpKind::Reduce: {
            const Spec& x = spec_of(in, 0);
            expect(dtype_is_float(x.dtype), "reduce only supports f32/bf16 tensors");
            if (in.a.size() != 1) fail_exec("reduce currently supports single axis");
            in.a[0] = norm_axis(in.a[0], x.rank(), "reduce");
            std::vector<int64_t> want;
            for (int i = 0; i < x.rank(); ++i) {
                if (i == in.a[0]) { if (in.keepdims) want.push_back(1); }
                else want.push_back(x.dims[i]);
            }
            expect(out.dtype == x.dtype && out.dims == want, "reduce output shape mismatch");
            break;
        }
        case OpKind::Dot: {
            const Spec& l = spec_of(in, 0);
            const Spec& r = spec_of(in, 1);
            expect(l.dtype == r.dtype && dtype_is_float(l.dtype), "dot_general only supports f32/bf16 tensors of one dtype");
            expect(in.a.size() == in.b.size(), "dot_general batch dimension mismatch");
            expect(in.c.size() == in.d.size(), "dot_general dimension mismatch");
            auto check_axes = [&](const std::vector<int64_t>& ax, int rank) {
                for (auto a : ax) expect(a >= 0 && a < rank, "dot_general axis out of range");
            };
            check_axes(in.a, l.rank()); check_axes(in.c, l.rank());
            check_axes(in.b, r.rank()); check_axes(in.d, r.rank());
            for (size_t i = 0; i < in.a.size(); ++i) expect(l.dims[in.a[i]] == r.dims[in.b[i]], "dot_general batch dimension mismatch");
            for (size_t i = 0; i < in.c.size(); ++i) expect(l.dims[in.c[i]] == r.dims[in.d[i]], "dot_general dimension mismatch on contraction");
            std::vector<int64_t> want;
            std::vector<int64_t> bl = in.a;
            std::sort(bl.begin(), bl.end());
            for (auto a : bl) want.push_back(l.dims[a]);
            auto has = [](const std::vector<int64_t>& v, int64_t x) { return std::find(v.begin(), v.end(), x) != v.end(); };
            for (int i = 0; i < l.rank(); ++i) if (!has(in.a, i) && !has(in.c, i)) want.push_back(l.dims[i]);
            for (int i = 0; i < r.rank(); ++i) if (!has(in.b, i) && !has(in.d, i)) want.push_back(r.dims[i]);
            // out_dtype = F32 on bf16 operands keeps the f32 accumulator (docs/backend.md:104-115)
            in.out_f32 = in.out_f32 && l.dtype == DType::BF16;
            expect((out.dtype == l.dtype || in.out_f32) && out.dims == want, "dot_general output shape mismatch");
            break;
        }
        case OpKind::CustomCall: {
            // Weight-only quantisation extension of this backend; its targets are validated here and become
            // FLinear(quant) / FQuant.  docs/backend.md:581-582: unknown targets MUST answer Unimplemented.
            const int qd = quant_dot_target(in.target), qo = quant_op_target(in.target);
            if (!qd && !qo) fail_unimpl("custom_call", "unknown target `" + in.target + "`");
            auto is_f = [](const Spec& sp) { return sp.dtype == DType::F32 || sp.dtype == DType::BF16; };
            // (codes, scales) of a [K,N] weight matrix in scheme q (1 int8 per column, 2 int4 groups of 128)
            auto check_pair = [&](int q, const Spec& codes, const Spec& scales, int64_t K, int64_t N, DType fdt) {
                if (q == 1) {
                    expect(codes.dtype == DType::SI8 && codes.dims == std::vector<int64_t>{K, N}, in.target + ": codes must be si8[K,N]");
                    expect(scales.dtype == fdt && scales.dims == std::vector<int64_t>{N}, in.target + ": scales must be [N] of the float dtype");
                } else {
                    expect(K % 128 == 0, in.target + ": K must be a multiple of the group size 128");
                    expect(codes.dtype == DType::UI8 && codes.dims == std::vector<int64_t>{K / 2, N}, in.target + ": codes must be ui8[K/2,N]");
                    expect(scales.dtype == fdt && scales.dims == std::vector<int64_t>{K / 128, N}, in.target + ": scales must be [K/128,N] of the float dtype");
                }
            };
            if (qd) {
                expect(in.operands.size() == 3, in.target + ": expects (x, codes, scales)");
                const Spec& x = spec_of(in, 0);
                expect(is_f(x) && x.rank() == 2, in.target + ": x must be a float matrix [M,K]");
                const Spec& c = spec_of(in, 1);
                expect(c.rank() == 2, in.target + ": codes must be a matrix");
                check_pair(qd, c, spec_of(in, 2), x.dims[1], c.dims[1], x.dtype);
                in.out_f32 = x.dtype == DType::BF16 && out.dtype == DType::F32;   // the accumulator leaves as f32
                expect((out.dtype == x.dtype || in.out_f32) && out.dims == std::vector<int64_t>{x.dims[0], c.dims[1]},
                       in.target + ": output must be [M,N] of x's dtype (or f32)");
                in.op = OpKind::FLinear;
                in.op_name = qd == 1 ? "fused.linear_w8" : "fused.linear_w4g128";
                in.quant = qd;
                in.act = 0;
                break;
            }
            const int scheme = (qo == 1 || qo == 2 || qo == 5) ? 1 : 2;
            if (qo == 1 || qo == 3) {          // scales(w)
                expect(in.operands.size() == 1, in.target + ": expects (w)");
                const Spec& w = spec_of(in, 0);
                expect(is_f(w) && w.rank() == 2, in.target + ": w must be a float matrix [K,N]");
                if (scheme == 2) expect(w.dims[0] % 128 == 0, in.target + ": K must be a multiple of the group size 128");
                const std::vector<int64_t> want = scheme == 1 ? std::vector<int64_t>{w.dims[1]} : std::vector<int64_t>{w.dims[0] / 128, w.dims[1]};
                expect(out.dtype == w.dtype && out.dims == want, in.target + ": output shape mismatch");
            } else if (qo == 2 || qo == 4) {   // codes(w, scales)
                expect(in.operands.size() == 2, in.target + ": expects (w, scales)");
                const Spec& w = spec_of(in, 0);
                expect(is_f(w) && w.rank() == 2, in.target + ": w must be a float matrix [K,N]");
                check_pair(scheme, out, spec_of(in, 1), w.dims[0], w.dims[1], w.dtype);
            } else {                           // dequantise(codes, scales)
                expect(in.operands.size() == 2, in.target + ": expects (codes, scales)");
                expect(is_f(out) && out.rank() == 2, in.target + ": output must be a float matrix [K,N]");
                check_pair(scheme, spec_of(in, 0), spec_of(in, 1), out.dims[0], out.dims[1], out.dtype);
            }
            in.op = OpKind::FQuant;
            in.op_name = "quant." + in.target;
            in.quant = qo;
            break;
        }
        case OpKind::Unsupported:
            fail_unimpl(in.op_name, "operation not supported in the hip backend");
        default:
            break;  // fused ops are produced from already-validated sequences
    }
}

// Element strides of `src` broadcast (right-aligned) to `out_rank` dims: 0 where it repeats.
static std::vector<int64_t> broadcast_strides(const Spec& src, const Spec& out) {
    std::vector<int64_t> s = row_major_strides(src.dims), r(out.rank(), 0);
    const int pad = out.rank() - src.rank();
    for (int i = 0; i < src.rank(); ++i) r[pad + i] = src.dims[i] == 1 ? 0 : s[i];
    return r;
}

// One group of dot axes as a single (extent, stride), or false when they do not collapse.
static bool collapse_axes(const Spec& s, const std::vector<int64_t>& axes, int64_t& extent, int64_t& stride) {
    const auto st = row_major_strides(s.dims);
    extent = 1;
    stride = 1;
    std::vector<std::pair<int64_t, int64_t>> ds;  // (dim, stride), skipping extent-1 axes
    for (auto a : axes) {
        extent *= s.dims[a];
        if (s.dims[a] != 1) ds.push_back({s.dims[a], st[a]});
    }
    if (ds.empty()) { stride = 0; return true; }
    for (size_t i = 0; i + 1 < ds.size(); ++i)
        if (ds[i].second != ds[i + 1].second * ds[i + 1].first) return false;
    stride = ds.back().second;
    return true;
}

void Builder::describe(Step& st) {
    Instr& in = st.in;
    const Spec& out = in.out_specs[0];
    const auto out_strides = row_major_strides(out.dims);
    auto es_of = [&](const Spec& s) { return (int)dtype_size(s.dtype); };
    switch (in.op) {
        case OpKind::BroadcastTo: {
            const Spec& x = spec_of(in, 0);
            st.copies.push_back(make_copy(out.dims, out_strides, broadcast_strides(x, out), 0, 0));
            st.elem_size = widen_copies(st.copies, es_of(out));
            break;
        }
        case OpKind::Slice: {
            const Spec& x = spec_of(in, 0);
            const auto xs = row_major_strides(x.dims);
            int64_t off = 0;
            for (int i = 0; i < x.rank(); ++i) off += in.a[i] * xs[i];
            st.copies.push_back(make_copy(out.dims, out_strides, xs, 0, off));
            st.elem_size = widen_copies(st.copies, es_of(out));
            break;
        }
        case OpKind::Transpose: {
            const Spec& x = spec_of(in, 0);
            const auto xs = row_major_strides(x.dims);
            std::vector<int64_t> ss(x.rank());
            for (int i = 0; i < x.rank(); ++i) ss[i] = xs[in.a[i]];
            st.copies.push_back(make_copy(out.dims, out_strides, ss, 0, 0));
            st.elem_size = widen_copies(st.copies, es_of(out));
            break;
        }
        case OpKind::Concat: {
            int64_t along = 0;
            for (size_t i = 0; i < in.operands.size(); ++i) {
                const Spec& x = spec_of(in, i);
                st.copies.push_back(make_copy(x.dims, out_strides, row_major_strides(x.dims), along * out_strides[in.axis], 0));
                along += x.dims[in.axis];
            }
            st.elem_size = widen_copies(st.copies, es_of(out));
            break;
        }
        case OpKind::DynamicSlice: {
            const Spec& x = spec_of(in, 0);
            const auto xs = row_major_strides(x.dims);
            k::CopyDesc c = make_copy(out.dims, out_strides, xs, 0, 0);
            c.dyn = 1;
            c.dyn_rank = x.rank();
            if (x.rank() > k::kMaxRank) fail_unimpl("dynamic_slice", "rank above 6");
            for (int i = 0; i < x.rank(); ++i) { c.dyn_max[i] = x.dims[i] - in.a[i]; c.dyn_stride[i] = c.dyn_max[i] ? xs[i] : 0; }
            st.copies.push_back(c);
            st.elem_size = widen_copies(st.copies, es_of(out));
            break;
        }
        case OpKind::DynamicUpdateSlice: {
            const Spec& x = spec_of(in, 0);
            // the update itself, or a view of operand 1 that the fusion pass composed (shape, strides, offset)
            const bool view = !in.view_dims.empty();
            const std::vector<int64_t> udims = view ? in.view_dims : spec_of(in, 1).dims;
            const auto xs = row_major_strides(x.dims);
            k::CopyDesc c = make_copy(udims, xs, view ? in.view_strides : row_major_strides(udims), 0, view ? in.view_off : 0);
            c.dyn = 2;
            c.dyn_rank = x.rank();
            if (x.rank() > k::kMaxRank) fail_unimpl("dynamic_update_slice", "rank above 6");
            for (int i = 0; i < x.rank(); ++i) { c.dyn_max[i] = x.dims[i] - udims[i]; c.dyn_stride[i] = c.dyn_max[i] ? xs[i] : 0; }
            st.copies.push_back(c);
            st.elem_size = widen_copies(st.copies, es_of(out));
            break;
        }
        case OpKind::Iota: {
            st.outer = 1; st.inner = 1;
            for (int i = 0; i < in.axis; ++i) st.outer *= out.dims[i];
            for (int i = (int)in.axis + 1; i < out.rank(); ++i) st.inner *= out.dims[i];
            st.axis_len = out.dims[in.axis];
            break;
        }
        case OpKind::Reduce: {
            const Spec& x = spec_of(in, 0);
            const int ax = (int)in.a[0];
            st.outer = 1; st.inner = 1;
            for (int i = 0; i < ax; ++i) st.outer *= x.dims[i];
            for (int i = ax + 1; i < x.rank(); ++i) st.inner *= x.dims[i];
            st.axis_len = x.dims[ax];
            break;
        }
        case OpKind::Take: {
            const Spec& x = spec_of(in, 0);
            st.outer = spec_of(in, 1).count();
            st.axis_len = x.dims[0];
            st.inner = x.dims[0] ? x.count() / x.dims[0] : 0;
            break;
        }
        case OpKind::Dot: {
            const Spec& l = spec_of(in, 0);
            const Spec& r = spec_of(in, 1);
            auto has = [](const std::vector<int64_t>& v, int64_t x) { return std::find(v.begin(), v.end(), x) != v.end(); };
            // batch axes sorted as the reference does (cpu.rs:2166-2169); pair them up accordingly
            std::vector<std::pair<int64_t, int64_t>> bp;
            for (size_t i = 0; i < in.a.size(); ++i) bp.push_back({in.a[i], in.b[i]});
            std::vector<int64_t> bl = in.a, br = in.b;
            std::sort(bl.begin(), bl.end());
            std::sort(br.begin(), br.end());
            std::vector<int64_t> lf, rf;
            for (int i = 0; i < l.rank(); ++i) if (!has(in.a, i) && !has(in.c, i)) lf.push_back(i);
            for (int i = 0; i < r.rank(); ++i) if (!has(in.b, i) && !has(in.d, i)) rf.push_back(i);
            k::DotDesc& d = st.dot;
            int64_t e;
            bool lok = collapse_axes(l, bl, d.batch, d.a_sb) & collapse_axes(l, lf, d.m, d.a_sm) & collapse_axes(l, in.c, d.k, d.a_sk);
            bool rok = collapse_axes(r, br, e, d.b_sb) & collapse_axes(r, in.d, e, d.b_sk) & collapse_axes(r, rf, d.n, d.b_sn);
            d.c_sb = d.m * d.n;
            d.c_sm = d.n;
            const size_t es = dtype_size(l.dtype);
            size_t scratch = 0;
            if (!lok) {  // repack lhs as [batch][m][k]
                std::vector<int64_t> order = bl;
                order.insert(order.end(), lf.begin(), lf.end());
                order.insert(order.end(), in.c.begin(), in.c.end());
                const auto ls = row_major_strides(l.dims);
                std::vector<int64_t> dims, ss;
                for (auto a : order) { dims.push_back(l.dims[a]); ss.push_back(ls[a]); }
                st.pack_l = make_copy(dims, row_major_strides(dims), ss, 0, 0);
                st.lhs_pack = true;
                st.pack_l_off = scratch;
                scratch += align_up((size_t)l.count() * es);
                d.a_sb = d.m * d.k; d.a_sm = d.k; d.a_sk = 1;
            }
            if (!rok) {  // repack rhs as [batch][k][n]
                std::vector<int64_t> order = br;
                order.insert(order.end(), in.d.begin(), in.d.end());
                order.insert(order.end(), rf.begin(), rf.end());
                const auto rs = row_major_strides(r.dims);
                std::vector<int64_t> dims, ss;
                for (auto a : order) { dims.push_back(r.dims[a]); ss.push_back(rs[a]); }
                st.pack_r = make_copy(dims, row_major_strides(dims), ss, 0, 0);
                st.rhs_pack = true;
                st.pack_r_off = scratch;
                scratch += align_up((size_t)r.count() * es);
                d.b_sb = d.k * d.n; d.b_sk = d.n; d.b_sn = 1;
            }
            st.scratch_bytes = scratch;
            break;
        }
        case OpKind::FLinear: {
            const Spec& x = spec_of(in, 0);
            const Spec& w = spec_of(in, 1);
            const DType ldt = linear_dtype(in, w, in.quant ? &spec_of(in, 2) : nullptr);
            if (in.tiled || in.mfma) {
                auto pos = [&](size_t op) {
                    const int v = in.operands[op].value;
                    const int p = v >= 0 && v < (int)param_pos.size() ? param_pos[v] : -1;
                    if (p < 0) fail_exec("tiled linear: weight operand is not a program input");
                    return p;
                };
                st.tiled_w_input = pos(1);
                if (in.act == 2) st.tiled_w2_input = pos(linear_w2_pos(in));
                if (in.quant) {
                    st.tiled_s_input = pos(2);
                    if (in.act == 2) st.tiled_s2_input = pos(4);
                }
            }
            if (in.mfma) st.scratch_bytes = k::mfma_workspace_bytes((int)ldt, x.dims[0], x.dims[1], w.dims[1], in.act == 2, in.quant);
            if (in.tiled && x.dims[0] >= 2) {
                // batched decode normalises into scratch first (the matrix-core kernel reads plain rows); layers with
                // few column tiles add the partial sums of their K splits
                st.scratch_bytes = align_up(in.norm ? (size_t)x.count() * dtype_size(x.dtype) : 0) +
                                   align_up(k::skinny_workspace_bytes(x.dims[1], w.dims[1], in.act == 2));
            }
            if (in.quant && !in.mfma && !(in.tiled && x.dims[0] >= 2)) {
                // stand-alone path of a quantised linear: (RMSNorm of x,) dequantised weights, then the generic kernel
                const size_t es = dtype_size(ldt);
                st.scratch_bytes = align_up(in.norm ? (size_t)x.count() * es : 0) +
                                   align_up((size_t)x.dims[1] * w.dims[1] * es) * (in.act == 2 ? 2 : 1) +
                                   k::linear_workspace_bytes((int)ldt, x.dims[0], x.dims[1], w.dims[1], in.act == 2);
            } else if (!in.tiled && !in.mfma) {
                st.scratch_bytes = k::linear_workspace_bytes((int)ldt, x.dims[0], x.dims[1], w.dims[1], in.act == 2);
            }
            break;
        }
        case OpKind::FAttnDecode: {
            const Spec& ck = spec_of(in, 1);
            st.scratch_bytes = std::max(k::attn_decode_workspace_bytes(in.n_q, in.head_dim, ck.dims[1]),
                                        k::chain_attn_part_bytes(in.n_q, in.n_kv, in.head_dim)) * (size_t)std::max<int64_t>(in.batch, 1);
            break;
        }
        default:
            break;
    }
}

void Builder::build() {
    Function& fn = plan.fn;
    plan.values.assign(fn.max_value_id + 1, ValueInfo{});
    if (fn.param_ids.size() != donated.size()) fail_exec("entry input arity mismatch");
    for (size_t i = 0; i < fn.param_ids.size(); ++i) define(fn.param_ids[i], fn.param_specs[i]);
    param_pos.assign(plan.values.size(), -1);
    for (size_t i = 0; i < fn.param_ids.size(); ++i) param_pos[fn.param_ids[i]] = (int)i;

    // literals -> const block
    lit_offset.resize(fn.literals.size());
    for (size_t i = 0; i < fn.literals.size(); ++i) lit_offset[i] = const_add(fn.literals[i].bytes);

    // pass 1: validate, define values, record aliasing
    for (auto& in : fn.body) {
        if (in.dead) continue;
        for (size_t i = 0; i < in.operands.size(); ++i) (void)spec_of(in, i);
        validate(in);
        for (size_t o = 0; o < in.out_ids.size(); ++o) define(in.out_ids[o], in.out_specs[o]);
        const bool alias = in.op == OpKind::Reshape || in.op == OpKind::StopGradient ||
                           (in.op == OpKind::Cast && spec_of(in, 0).dtype == in.out_specs[0].dtype);
        if (alias && in.operands[0].value >= 0) plan.values[in.out_ids[0]].root = root(in.operands[0].value);
    }
    for (size_t i = 0; i < fn.result_ids.size(); ++i) {
        const int id = fn.result_ids[i];
        if (id < 0 || id >= (int)plan.values.size() || !plan.values[id].defined) fail_exec("missing function result value");
        if (plan.values[id].spec != fn.result_specs[i]) fail_exec("function result spec mismatch");
    }

    // pass 2: steps
    const int nv = (int)plan.values.size();
    use_count.assign(nv, 0);
    last_use.assign(nv, -1);
    def_step.assign(nv, -1);
    plan.storage.assign(nv, RootStorage{});
    for (auto& in : fn.body) {
        if (in.dead) continue;
        const bool alias = plan.values[in.out_ids[0]].root != in.out_ids[0];
        if (in.op == OpKind::Constant) {
            RootStorage& rs = plan.storage[in.out_ids[0]];
            rs.kind = Storage::Const;
            rs.offset = lit_offset[in.literal];
            continue;
        }
        if (alias) continue;  // pure view: no work
        Step st;
        st.in = in;
        for (auto& o : in.operands) {
            st.src.push_back(o.value);
            st.src_const.push_back(o.value < 0 ? lit_offset[o.literal] : 0);
        }
        st.dst = in.out_ids;
        describe(st);
        const int idx = (int)plan.steps.size();
        for (int v : st.src)
            if (v >= 0) { const int r = root(v); ++use_count[r]; last_use[r] = idx; }
        for (int v : st.dst) def_step[v] = idx;
        plan.steps.push_back(std::move(st));
    }
    const int n_steps = (int)plan.steps.size();

    // storage classes
    for (size_t i = 0; i < fn.param_ids.size(); ++i) {
        RootStorage& rs = plan.storage[fn.param_ids[i]];
        rs.kind = Storage::Input;
        rs.index = (int)i;
    }
    std::vector<int> input_of_root(nv, -1);
    for (size_t i = 0; i < fn.param_ids.size(); ++i) input_of_root[fn.param_ids[i]] = (int)i;
    std::vector<bool> root_is_result(nv, false);
    for (int id : fn.result_ids) root_is_result[root(id)] = true;

    // results -> output buffers (shared when several results alias one root)
    std::map<int, int> out_buf_of_root;
    plan.out_buffer_of_result.assign(fn.result_ids.size(), -1);
    plan.result_input_alias.assign(fn.result_ids.size(), -1);
    auto new_out_buffer = [&](int r) {
        const int ob = (int)plan.out_buffer_bytes.size();
        plan.out_buffer_bytes.push_back(std::max<size_t>(plan.values[r].spec.bytes(), 1));
        plan.out_buffer_inplace_input.push_back(-1);
        out_buf_of_root[r] = ob;
        plan.storage[r].kind = Storage::Output;
        plan.storage[r].index = ob;
        return ob;
    };
    for (size_t i = 0; i < fn.result_ids.size(); ++i) {
        const int r = root(fn.result_ids[i]);
        if (plan.storage[r].kind == Storage::Input) { plan.result_input_alias[i] = plan.storage[r].index; continue; }
        if (plan.storage[r].kind == Storage::Const) {
            // a constant returned directly: give it an output buffer filled by a copy step
            fail_unimpl("constant", "returning a Constant as a function result");
        }
        auto it = out_buf_of_root.find(r);
        plan.out_buffer_of_result[i] = it != out_buf_of_root.end() ? it->second : new_out_buffer(r);
    }

    // in-place updates on donated inputs
    for (auto& st : plan.steps) {
        std::vector<std::pair<int, int>> pairs;  // (base operand slot, output slot)
        if (st.in.op == OpKind::DynamicUpdateSlice) pairs = {{0, 0}};
        if (st.in.op == OpKind::FAttnDecode)
            for (int64_t b = 0; b < std::max<int64_t>(st.in.batch, 1); ++b) {
                pairs.push_back({(int)attn_cache_operand(st.in, b), (int)attn_cache_output(b)});
                pairs.push_back({(int)attn_cache_operand(st.in, b) + 1, (int)attn_cache_output(b) + 1});
            }
        bool all_inplace = !pairs.empty();
        for (auto& pr : pairs) {
            const int bv = st.src[pr.first];
            bool ok = bv >= 0;
            int br = ok ? root(bv) : -1;
            ok = ok && input_of_root[br] >= 0 && donated[input_of_root[br]] && use_count[br] == 1 && !root_is_result[br];
            const int ov = st.dst[pr.second];
            ok = ok && plan.storage[ov].kind == Storage::Output;  // the updated cache is a program result
            if (ok) {
                // a second in-place claim on one input would alias two outputs
                for (int ip : plan.out_buffer_inplace_input) ok = ok && ip != input_of_root[br];
            }
            if (ok) {
                plan.out_buffer_inplace_input[plan.storage[ov].index] = input_of_root[br];
            } else {
                all_inplace = false;
            }
        }
        st.copy_base = !all_inplace;  // informational: run_step compares pointers
    }

    // workspace: temps by liveness (first-fit over a free list), plus per-step scratch
    struct Block { size_t off, size; };
    std::vector<Block> free_list;
    size_t high = 0;
    auto ws_alloc = [&](size_t bytes) {
        bytes = align_up(std::max<size_t>(bytes, 1));
        for (size_t i = 0; i < free_list.size(); ++i) {
            if (free_list[i].size >= bytes) {
                const size_t off = free_list[i].off;
                free_list[i].off += bytes;
                free_list[i].size -= bytes;
                if (!free_list[i].size) free_list.erase(free_list.begin() + i);
                return off;
            }
        }
        const size_t off = high;
        high += bytes;
        return off;
    };
    auto ws_free = [&](size_t off, size_t bytes) {
        bytes = align_up(std::max<size_t>(bytes, 1));
        free_list.push_back({off, bytes});
        std::sort(free_list.begin(), free_list.end(), [](const Block& a, const Block& b) { return a.off < b.off; });
        for (size_t i = 0; i + 1 < free_list.size();) {
            if (free_list[i].off + free_list[i].size == free_list[i + 1].off) {
                free_list[i].size += free_list[i + 1].size;
                free_list.erase(free_list.begin() + i + 1);
            } else {
                ++i;
            }
        }
    };
    std::vector<std::vector<int>> dying(n_steps);
    for (int v = 0; v < nv; ++v)
        if (plan.values[v].defined && plan.values[v].root == v && def_step[v] >= 0 && plan.storage[v].kind == Storage::Temp)
            dying[std::max(last_use[v], def_step[v])].push_back(v);
    for (int s = 0; s < n_steps; ++s) {
        Step& st = plan.steps[s];
        for (int v : st.dst) {
            RootStorage& rs = plan.storage[v];
            if (rs.kind != Storage::Temp) continue;
            rs.bytes = std::max<size_t>(plan.values[v].spec.bytes(), 1);
            rs.offset = ws_alloc(rs.bytes);
        }
        if (st.scratch_bytes) {
            st.scratch_off = ws_alloc(st.scratch_bytes);
            ws_free(st.scratch_off, st.scratch_bytes);
        }
        for (int v : dying[s]) ws_free(plan.storage[v].offset, plan.storage[v].bytes);
    }
    plan.workspace_bytes = high;

    // runs of consecutive decode linears / decode attentions -> one persistent launch each
    auto chain_phases = [&](const Step& st) -> int {   // phases the step takes in a chain, 0: not chainable
        const Instr& in = st.in;
        if (in.op == OpKind::FAttnDecode) {
            if (in.batch > 1) return 0;
            const Spec& x = plan.values[st.src[0]].spec;
            if (!k::chain_attn_supported((int)x.dtype, x.dims[0], in.n_q, in.n_kv, in.head_dim, in.rot_half)) return 0;
            return k::chain_attn_phases(plan.values[st.src[1]].spec.dims[1]);
        }
        if (in.op != OpKind::FLinear || !in.tiled || st.tiled_w_input < 0) return 0;
        const Spec& x = plan.values[st.src[0]].spec;
        const Spec& w = plan.values[st.src[1]].spec;
        if (x.rank() != 2 || w.rank() != 2) return 0;
        const bool dual = in.act == 2;
        const DType ldt = linear_dtype(in, w, in.quant ? &plan.values[st.src[2]].spec : nullptr);
        const int wfmt = chain_format(in, ldt);
        if (in.norm_ln && wfmt != k::kChainW32) return 0;   // LayerNorm is staged for f32 phases only
        if (wfmt == k::kChainW32 && (in.norm && !in.norm_ln)) return 0;   // ... and RMSNorm for the others
        if (!k::chain_supported((int)ldt, x.dims[0], x.dims[1], w.dims[1], dual, in.norm, wfmt, in.x_f32, !in.has_bias && !in.has_residual)) return 0;
        k::ChainPhase p{};
        return k::chain_fill_phase(p, x.dims[1], w.dims[1], dual, wfmt) ? 1 : 0;
    };
    auto step_format = [&](const Step& st) {
        const Instr& in = st.in;
        const Spec& w = plan.values[st.src[1]].spec;
        return chain_format(in, linear_dtype(in, w, in.quant ? &plan.values[st.src[2]].spec : nullptr));
    };
    // f32 linears and f32 attentions go together (the launch's kernel reads f32 rows and caches), the others likewise
    auto f32_class = [&](const Step& st) {
        if (st.in.op == OpKind::FAttnDecode) return plan.values[st.src[0]].spec.dtype == DType::F32;
        return step_format(st) == k::kChainW32;
    };
    for (int s = 0; s < n_steps;) {
        int np = chain_phases(plan.steps[s]);
        if (!np) { ++s; continue; }
        int e = s + 1;
        bool has_linear = plan.steps[s].in.op == OpKind::FLinear;
        int fmt = has_linear ? step_format(plan.steps[s]) : -1;   // one weight format per launch
        const bool cls = f32_class(plan.steps[s]);
        while (e < n_steps) {
            const Step& nx = plan.steps[e];
            const int q = chain_phases(nx);
            if (!q || np + q > k::kChainMaxPhases) break;
            if (f32_class(nx) != cls) break;
            if (nx.in.op == OpKind::FLinear) {
                if (fmt >= 0 && step_format(nx) != fmt) break;
                fmt = step_format(nx);
                has_linear = true;
            }
            np += q;
            ++e;
        }
        if (has_linear) {   // an attention on its own keeps its stand-alone kernels
            plan.steps[s].chain_len = e - s;
            for (int i = s + 1; i < e; ++i) plan.steps[i].chain_member = true;
        }
        s = e;
    }
}

void build_plan(Plan& plan, const std::vector<bool>& donated) {
    Builder b(plan, donated);
    b.build();
}

// ------------------------------------------------------------------------------ execution
static inline const void* src_ptr(const Step& st, const ExecCtx& cx, size_t i) {
    return st.src[i] >= 0 ? cx.ptr[st.src[i]] : (const void*)(cx.consts + st.src_const[i]);
}

// algorithmic bytes of the weights an FLinear reads once: codes and scales when quantised
static int64_t linear_weight_bytes(const Instr& in, DType ldt, const Spec& x, const Spec& w) {
    const int64_t K = x.dims[1], N = w.dims[1], es = (int64_t)dtype_size(ldt);
    int64_t b = in.quant == 0 ? K * N * es : (in.quant == 1 ? K * N + N * es : K * N / 2 + (K / 128) * N * es);
    return b * (in.act == 2 ? 2 : 1);
}

// One persistent launch for the steps [st, st + chain_len): builds the phase table from the resolved
// pointers, fetches its cached device copy and launches.  false: the caller runs the steps one by one
// (cx.chain is cleared so the members run too).
static bool run_chain(const Plan& plan, const Step& head, ExecCtx& cx) {
    std::vector<k::ChainPhase> phases;
    phases.reserve((size_t)head.chain_len * 2);
    int lds_bytes = 0, wfmt = k::kChainW16;
    int64_t bytes = 0;
    auto aligned8 = [](std::initializer_list<const void*> ps) {
        for (const void* q : ps) if ((uintptr_t)q & 7) fail_exec("decode chain: operand buffers must be 8-byte aligned");
    };
    {   // f32 phases pay off once they have something to stream (Backend::chain_f32_min_bytes)
        int64_t f32_bytes = 0, f32_linears = 0;
        for (int i = 0; i < head.chain_len; ++i) {
            const Step& st = (&head)[i];
            if (st.in.op != OpKind::FLinear) continue;
            const Spec& x = plan.values[st.src[0]].spec;
            const Spec& w = plan.values[st.src[1]].spec;
            if (chain_format(st.in, linear_dtype(st.in, w, st.in.quant ? &plan.values[st.src[2]].spec : nullptr)) != k::kChainW32) continue;
            f32_bytes += x.dims[1] * w.dims[1] * 4;
            ++f32_linears;
        }
        if (f32_linears > 0 && f32_bytes < cx.be->chain_f32_min_bytes * f32_linears) { cx.chain = false; return false; }
    }
    for (int i = 0; i < head.chain_len; ++i) {
        const Step& st = (&head)[i];
        const Instr& in = st.in;
        if (in.op == OpKind::FAttnDecode) {
            const Spec& ck = plan.values[st.src[1]].spec;
            void* kout = cx.ptr[st.dst[1]];
            void* vout = cx.ptr[st.dst[2]];
            const void* kin = src_ptr(st, cx, 1);
            const void* vin = src_ptr(st, cx, 2);
            // caches that were not donated are copied ahead of the launch (they are inputs of the run)
            if (kout != kin) { GPTRS_HIP_CHECK(hipMemcpyAsync(kout, kin, ck.bytes(), hipMemcpyDeviceToDevice, cx.stream)); ++cx.launches; }
            if (vout != vin) { GPTRS_HIP_CHECK(hipMemcpyAsync(vout, vin, ck.bytes(), hipMemcpyDeviceToDevice, cx.stream)); ++cx.launches; }
            k::ChainPhase pa{}, pc{};
            k::chain_fill_attn(pa, pc, in.n_q, in.n_kv, in.head_dim, ck.dims[1], in.rot_half, in.scale);
            pa.x = src_ptr(st, cx, 0);
            pa.k_cache = kout; pa.v_cache = vout;
            pa.update_starts = (const int32_t*)src_ptr(st, cx, 3);
            pa.query_start = (const int32_t*)src_ptr(st, cx, 4);
            if (in.rot_half > 0) { pa.cos = src_ptr(st, cx, 5); pa.sin = src_ptr(st, cx, 6); }
            pa.part = (float*)(cx.ws + st.scratch_off);
            pc.part = pa.part;
            pc.y = cx.ptr[st.dst[0]];
            pa.y = pc.y;   // (written by the first phase when it is the only one)
            aligned8({pa.x, pa.part, pc.y});
            if (((uintptr_t)kout | (uintptr_t)vout | (uintptr_t)pa.cos | (uintptr_t)pa.sin) & 15)
                fail_exec("decode chain: cache and RoPE buffers must be 16-byte aligned");
            const bool two = k::chain_attn_phases(ck.dims[1]) == 2;
            lds_bytes = std::max(lds_bytes, two ? std::max(pa.lds_total, pc.lds_total) : pa.lds_total);
            phases.push_back(pa);
            if (two) phases.push_back(pc);
            continue;
        }
        const Spec& x = plan.values[st.src[0]].spec;
        const Spec& w = plan.values[st.src[1]].spec;
        const bool dual = in.act == 2;
        k::ChainPhase p{};
        const DType ldt = linear_dtype(in, w, in.quant ? &plan.values[st.src[2]].spec : nullptr);
        wfmt = chain_format(in, ldt);
        if (!k::chain_fill_phase(p, x.dims[1], w.dims[1], dual, wfmt)) { cx.chain = false; return false; }
        BufferP wc = cx.be->derived_weights(cx.input_bufs[st.tiled_w_input], wfmt == k::kChainW32 ? 11 : (in.quant == 0 ? 2 : (in.quant == 1 ? 3 : 4)), ldt,
                                            x.dims[1], w.dims[1], dual ? cx.input_bufs[st.tiled_w2_input] : nullptr);
        p.w = wc->ptr;
        p.x = src_ptr(st, cx, 0);
        if (in.quant == 1) {         // per-column scales are read as they are
            p.wscale = src_ptr(st, cx, 2);
            if (dual) p.wscale2 = src_ptr(st, cx, 4);
            if (((uintptr_t)p.wscale | (uintptr_t)p.wscale2) & 3) fail_exec("decode chain: scale buffers must be 4-byte aligned");
        } else if (in.quant == 2) {  // group scales follow the tile order of the weights
            BufferP sc = cx.be->derived_weights(cx.input_bufs[st.tiled_s_input], 5, ldt, x.dims[1], w.dims[1],
                                                dual ? cx.input_bufs[st.tiled_s2_input] : nullptr);
            p.wscale = sc->ptr;
        }
        size_t oi = linear_extra_pos(in);
        if (in.has_bias) { p.bias = src_ptr(st, cx, oi++); p.flags |= k::kChainBias; }
        if (in.has_residual) { p.residual = src_ptr(st, cx, oi++); p.flags |= k::kChainResidual; }
        if (in.norm) { p.gamma = src_ptr(st, cx, oi++); p.inv_n = in.scale; p.eps = in.eps; p.flags |= k::kChainNorm; }
        if (in.norm && in.norm_ln) { p.beta = src_ptr(st, cx, oi++); p.flags |= k::kChainLayerNorm; }
        if (in.act == 1) p.flags |= k::kChainGelu;
        if (in.out_f32 || wfmt == k::kChainW32) p.flags |= k::kChainOutF32;
        if (in.x_f32 || wfmt == k::kChainW32) p.flags |= k::kChainXF32;
        p.y = cx.ptr[st.dst[0]];
        aligned8({p.x, p.y, p.residual, p.bias, p.gamma, p.beta});
        if ((p.flags & k::kChainXF32) && (((uintptr_t)p.gamma | (uintptr_t)p.beta | (uintptr_t)p.x) & 15))
            fail_exec("decode chain: f32 rows, gains and offsets must be 16-byte aligned");
        lds_bytes = std::max(lds_bytes, p.lds_total);
        bytes += (int64_t)dtype_size(x.dtype) * x.dims[1] + (int64_t)(in.out_f32 ? 4 : dtype_size(ldt)) * w.dims[1] + linear_weight_bytes(in, ldt, x, w);
        phases.push_back(p);
    }
    const k::ChainPhase* table = cx.be->chain_table(phases);
    if (!table) { cx.chain = false; return false; }
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (cx.profile) {
        GPTRS_HIP_CHECK(hipEventCreate(&e0));
        GPTRS_HIP_CHECK(hipEventCreate(&e1));
        GPTRS_HIP_CHECK(hipEventRecord(e0, cx.stream));
    }
    // a requested stall (a test hook) is consumed by the first launch that has a barrier to stall at
    int stall = -1;
    if (cx.be->chain_stall_phase >= 1 && phases.size() >= 2) {
        stall = std::min(cx.be->chain_stall_phase, (int)phases.size() - 1);
        cx.be->chain_stall_phase = -1;
        cx.be->chain_stall_fired = true;
    }
    if (!k::chain_launch(cx.stream, table, (int)phases.size(), lds_bytes, cx.be->chain_barrier(), cx.be->chain_abort_flag(), wfmt, stall)) {
        if (e0) { (void)hipEventDestroy(e0); (void)hipEventDestroy(e1); }
        cx.chain = false;
        return false;
    }
    if (cx.profile) {
        GPTRS_HIP_CHECK(hipEventRecord(e1, cx.stream));
        cx.be->prof_events.emplace_back(e0, e1);
        ++cx.be->prof_linear_calls;
        cx.be->prof_linear_bytes += bytes;
    }
    ++cx.be->n_chain_launches;
    cx.be->n_chain_phases += (int64_t)phases.size();
    ++cx.launches;
    return true;
}

void run_step(const Plan& plan, const Step& st, ExecCtx& cx) {
    const Instr& in = st.in;
    const Spec& out = in.out_specs[0];
    void* dst = cx.ptr[st.dst[0]];
    hipStream_t s = cx.stream;
    auto in_spec = [&](size_t i) -> const Spec& {
        return st.src[i] >= 0 ? plan.values[st.src[i]].spec : plan.fn.literals[in.operands[i].literal].spec;
    };
    switch (in.op) {
        case OpKind::BroadcastTo:
        case OpKind::Slice:
        case OpKind::Transpose:
            k::copy_strided(s, dst, src_ptr(st, cx, 0), st.elem_size, st.copies[0], nullptr);
            ++cx.launches;
            break;
        case OpKind::Concat:
            for (size_t i = 0; i < st.copies.size(); ++i) {
                k::copy_strided(s, dst, src_ptr(st, cx, i), st.elem_size, st.copies[i], nullptr);
                ++cx.launches;
            }
            break;
        case OpKind::DynamicSlice:
            k::copy_strided(s, dst, src_ptr(st, cx, 0), st.elem_size, st.copies[0], (const int32_t*)src_ptr(st, cx, 1));
            ++cx.launches;
            break;
        case OpKind::DynamicUpdateSlice: {
            const void* base = src_ptr(st, cx, 0);
            if (dst != base && out.bytes()) {
                GPTRS_HIP_CHECK(hipMemcpyAsync(dst, base, out.bytes(), hipMemcpyDeviceToDevice, s));
                ++cx.launches;
            }
            k::copy_strided(s, dst, src_ptr(st, cx, 1), st.elem_size, st.copies[0], (const int32_t*)src_ptr(st, cx, 2));
            ++cx.launches;
            break;
        }
        case OpKind::Unary:
            k::unary(s, (int)out.dtype, (int)in.unary, src_ptr(st, cx, 0), dst, out.count());
            ++cx.launches;
            break;
        case OpKind::Binary:
            if (in.scalar_rhs) k::binary_scalar(s, (int)out.dtype, (int)in.binary, src_ptr(st, cx, 0), in.scalar_val, dst, out.count());
            else k::binary(s, (int)out.dtype, (int)in.binary, src_ptr(st, cx, 0), src_ptr(st, cx, 1), dst, out.count());
            ++cx.launches;
            break;
        case OpKind::Compare:
            k::compare(s, (int)in_spec(0).dtype, (int)in.cmp, src_ptr(st, cx, 0), src_ptr(st, cx, 1), (uint8_t*)dst, out.count());
            ++cx.launches;
            break;
        case OpKind::Select:
            k::select(s, (int)dtype_size(out.dtype), (const uint8_t*)src_ptr(st, cx, 0), src_ptr(st, cx, 1), src_ptr(st, cx, 2), dst, out.count());
            ++cx.launches;
            break;
        case OpKind::Cast:
            k::cast(s, (int)in_spec(0).dtype, (int)out.dtype, src_ptr(st, cx, 0), dst, out.count());
            ++cx.launches;
            break;
        case OpKind::Iota:
            k::iota(s, (int32_t*)dst, st.outer, st.axis_len, st.inner);
            ++cx.launches;
            break;
        case OpKind::Reduce:
            k::reduce(s, (int)out.dtype, (int)in.reduce, src_ptr(st, cx, 0), dst, st.outer, st.axis_len, st.inner);
            ++cx.launches;
            break;
        case OpKind::Take:
            k::take(s, (int)dtype_size(out.dtype), src_ptr(st, cx, 0), (const int32_t*)src_ptr(st, cx, 1), dst, st.outer,
                    st.axis_len, st.inner, cx.err_flag);
            ++cx.launches;
            break;
        case OpKind::Dot: {
            const void* a = src_ptr(st, cx, 0);
            const void* b = src_ptr(st, cx, 1);
            const DType idt = in_spec(0).dtype;   // the operands' dtype (the result's may be f32 over bf16 operands)
            const int es = (int)dtype_size(idt);
            if (st.lhs_pack) {
                void* p = cx.ws + st.scratch_off + st.pack_l_off;
                k::copy_strided(s, p, a, es, st.pack_l, nullptr);
                a = p;
                ++cx.launches;
            }
            if (st.rhs_pack) {
                void* p = cx.ws + st.scratch_off + st.pack_r_off;
                k::copy_strided(s, p, b, es, st.pack_r, nullptr);
                b = p;
                ++cx.launches;
            }
            k::dot_generic(s, (int)idt, a, b, dst, st.dot, in.out_f32);
            ++cx.launches;
            break;
        }
        case OpKind::FLayerNorm: {
            const Spec& x = in_spec(0);
            const int64_t n = x.dims.back();
            k::layer_norm(s, (int)out.dtype, src_ptr(st, cx, 0), src_ptr(st, cx, 1), src_ptr(st, cx, 2), dst, n ? x.count() / n : 0, n, in.scale, in.eps);
            ++cx.launches;
            break;
        }
        case OpKind::FRmsNorm: {
            const Spec& x = in_spec(0);
            const int64_t n = x.dims.back();
            if (x.dtype == DType::F32 && out.dtype == DType::BF16)   // Cast(bf16)(rms_norm(x f32)) folded
                k::rms_norm_f32_to_bf16(s, src_ptr(st, cx, 0), src_ptr(st, cx, 1), dst, n ? x.count() / n : 0, n, in.scale, in.eps);
            else
                k::rms_norm(s, (int)out.dtype, src_ptr(st, cx, 0), src_ptr(st, cx, 1), dst, n ? x.count() / n : 0, n, in.scale, in.eps);
            ++cx.launches;
            break;
        }
        case OpKind::FSoftmax: {
            const int64_t n = out.dims.back();
            k::softmax_rows(s, (int)out.dtype, src_ptr(st, cx, 0), dst, n ? out.count() / n : 0, n);
            ++cx.launches;
            break;
        }
        case OpKind::FGelu:
            k::gelu(s, (int)out.dtype, src_ptr(st, cx, 0), dst, out.count(), in.fparam[0], in.fparam[1], in.fparam[2]);
            ++cx.launches;
            break;
        case OpKind::FSilu:
            k::swiglu(s, (int)out.dtype, src_ptr(st, cx, 0), nullptr, dst, out.count());
            ++cx.launches;
            break;
        case OpKind::FSwiglu:
            k::swiglu(s, (int)out.dtype, src_ptr(st, cx, 0), src_ptr(st, cx, 1), dst, out.count());
            ++cx.launches;
            break;
        case OpKind::FLinear: {
            if (cx.chain && st.chain_member) break;  // executed by the launch of the run's first step
            if (cx.chain && st.chain_len > 0 && run_chain(plan, st, cx)) break;
            const Spec& x = in_spec(0);
            const Spec& w = in_spec(1);
            const DType ldt = linear_dtype(in, w, in.quant ? &in_spec(2) : nullptr);
            const int64_t io_bytes = (int64_t)dtype_size(x.dtype) * x.count() + (int64_t)dtype_size(out.dtype) * out.count();
            // RMSNorm of x into scratch for the kernels that read plain rows of the compute dtype
            auto norm_into = [&](const void* xp, const void* gp, void* to) {
                if (in.x_f32) k::rms_norm_f32_to_bf16(s, xp, gp, to, x.dims[0], x.dims[1], in.scale, in.eps);
                else k::rms_norm(s, (int)ldt, xp, gp, to, x.dims[0], x.dims[1], in.scale, in.eps);
                ++cx.launches;
            };
            if (in.mfma) {
                k::MfmaLinearArgs ma{};
                ma.dtype = (int)ldt;
                ma.out_f32 = in.out_f32;
                ma.lds_direct = cx.be->opt_gemm_lds_direct ? 1 : 0;
                ma.x = src_ptr(st, cx, 0);
                ma.m = x.dims[0]; ma.k = x.dims[1]; ma.n = w.dims[1];
                // quantised weights: the k-grouped copy holds the codes; the kernel applies the scales on the way into LDS
                const int kind = in.quant == 0 ? 1 : (in.quant == 1 ? 6 : 7);
                BufferP wk = cx.be->derived_weights(cx.input_bufs[st.tiled_w_input], kind, ldt, ma.k, ma.n);
                BufferP wk2;
                ma.wk = wk->ptr;
                ma.quant = in.quant;
                if (in.quant) ma.scale = cx.input_bufs[st.tiled_s_input]->ptr;
                size_t oi = linear_extra_pos(in);
                if (in.act == 2) {
                    wk2 = cx.be->derived_weights(cx.input_bufs[st.tiled_w2_input], kind, ldt, ma.k, ma.n);
                    ma.wk2 = wk2->ptr;
                    if (in.quant) ma.scale2 = cx.input_bufs[st.tiled_s2_input]->ptr;
                }
                if (in.has_bias) ma.bias = src_ptr(st, cx, oi++);
                if (in.has_residual) ma.residual = src_ptr(st, cx, oi++);
                ma.y = dst;
                ma.act = in.act == 1 ? 1 : 0;
                if (st.scratch_bytes) {
                    ma.part = cx.ws + st.scratch_off;
                    ma.part_bytes = st.scratch_bytes;
                    ma.tickets = cx.be->skinny_tickets();
                }
                hipEvent_t e0 = nullptr, e1 = nullptr;
                if (cx.profile) {
                    GPTRS_HIP_CHECK(hipEventCreate(&e0));
                    GPTRS_HIP_CHECK(hipEventCreate(&e1));
                    GPTRS_HIP_CHECK(hipEventRecord(e0, s));
                }
                k::mfma_gemm(s, ma);
                if (cx.profile) {
                    GPTRS_HIP_CHECK(hipEventRecord(e1, s));
                    cx.be->prof_events.emplace_back(e0, e1);
                    ++cx.be->prof_linear_calls;
                    cx.be->prof_linear_bytes += io_bytes + linear_weight_bytes(in, ldt, x, w);
                }
                ++cx.launches;
                break;
            }
            if (in.tiled &&
                (in.quant ? k::skinny_quant_supported((int)ldt, x.dims[0], x.dims[1], w.dims[1], in.quant)
                          : k::skinny_gemm_supported((int)ldt, x.dims[0], x.dims[1], w.dims[1])) &&
                (!in.norm || st.scratch_bytes >= (size_t)x.count() * dtype_size(x.dtype))) {
                k::SkinnyLinearArgs sa{};
                sa.dtype = (int)ldt;
                sa.out_f32 = in.out_f32;
                sa.x = src_ptr(st, cx, 0);
                sa.m = x.dims[0]; sa.k = x.dims[1]; sa.n = w.dims[1];
                const int kind = in.quant == 0 ? 8 : (in.quant == 1 ? 9 : 10);   // bf16 copy, or the codes in the same tile order
                BufferP wsk = cx.be->derived_weights(cx.input_bufs[st.tiled_w_input], kind, ldt, sa.k, sa.n);
                BufferP wsk2;
                sa.ws = wsk->ptr;
                sa.quant = in.quant;
                if (in.quant) sa.scale = src_ptr(st, cx, 2);
                size_t oi = linear_extra_pos(in);
                if (in.act == 2) {
                    wsk2 = cx.be->derived_weights(cx.input_bufs[st.tiled_w2_input], kind, ldt, sa.k, sa.n);
                    sa.ws2 = wsk2->ptr;
                    if (in.quant) sa.scale2 = src_ptr(st, cx, 4);
                }
                if (in.has_bias) sa.bias = src_ptr(st, cx, oi++);
                if (in.has_residual) sa.residual = src_ptr(st, cx, oi++);
                const size_t norm_bytes = in.norm ? align_up((size_t)x.count() * dtype_size(x.dtype)) : 0;
                if (in.norm) {
                    void* xn = cx.ws + st.scratch_off;
                    if (in.norm_ln) {
                        k::layer_norm(s, (int)ldt, sa.x, src_ptr(st, cx, oi), src_ptr(st, cx, oi + 1), xn, sa.m, sa.k, in.scale, in.eps);
                        oi += 2;
                        ++cx.launches;
                    } else {
                        norm_into(sa.x, src_ptr(st, cx, oi++), xn);
                    }
                    sa.x = xn;
                }
                if (st.scratch_bytes > norm_bytes) {
                    sa.part = cx.ws + st.scratch_off + norm_bytes;
                    sa.part_bytes = st.scratch_bytes - norm_bytes;
                    sa.tickets = cx.be->skinny_tickets();
                }
                sa.y = dst;
                sa.act = in.act == 1 ? 1 : 0;
                hipEvent_t e0 = nullptr, e1 = nullptr;
                if (cx.profile) {
                    GPTRS_HIP_CHECK(hipEventCreate(&e0));
                    GPTRS_HIP_CHECK(hipEventCreate(&e1));
                    GPTRS_HIP_CHECK(hipEventRecord(e0, s));
                }
                k::skinny_gemm(s, sa);
                if (cx.profile) {
                    GPTRS_HIP_CHECK(hipEventRecord(e1, s));
                    cx.be->prof_events.emplace_back(e0, e1);
                    ++cx.be->prof_linear_calls;
                    cx.be->prof_linear_bytes += io_bytes + linear_weight_bytes(in, ldt, x, w);
                }
                ++cx.launches;
                break;
            }
            if (in.tiled && !in.quant) {
                k::TiledLinearArgs ta{};
                ta.dtype = (int)ldt;
                ta.out_f32 = in.out_f32;
                ta.x_f32 = in.x_f32;
                ta.x = src_ptr(st, cx, 0);
                ta.m = x.dims[0]; ta.k = x.dims[1]; ta.n = w.dims[1];
                BufferP wt = cx.be->derived_weights(cx.input_bufs[st.tiled_w_input], 0, ldt, ta.k, ta.n);
                BufferP wt2;
                ta.wt = wt->ptr;
                size_t oi = 2;
                if (in.act == 2) {
                    wt2 = cx.be->derived_weights(cx.input_bufs[st.tiled_w2_input], 0, ldt, ta.k, ta.n);
                    ta.wt2 = wt2->ptr;
                    ++oi;
                }
                if (in.has_bias) ta.bias = src_ptr(st, cx, oi++);
                if (in.has_residual) ta.residual = src_ptr(st, cx, oi++);
                if (in.norm) { ta.gamma = src_ptr(st, cx, oi++); ta.inv_n = in.scale; ta.eps = in.eps; }
                if (in.norm_ln) ta.beta = src_ptr(st, cx, oi++);
                ta.y = dst;
                ta.act = in.act == 1 ? 1 : 0;
                hipEvent_t e0 = nullptr, e1 = nullptr;
                if (cx.profile) {
                    GPTRS_HIP_CHECK(hipEventCreate(&e0));
                    GPTRS_HIP_CHECK(hipEventCreate(&e1));
                    GPTRS_HIP_CHECK(hipEventRecord(e0, s));
                }
                k::gemv_tiled(s, ta);
                if (cx.profile) {
                    GPTRS_HIP_CHECK(hipEventRecord(e1, s));
                    cx.be->prof_events.emplace_back(e0, e1);
                    ++cx.be->prof_linear_calls;
                    cx.be->prof_linear_bytes += io_bytes + linear_weight_bytes(in, ldt, x, w);
                }
                ++cx.launches;
                break;
            }
            k::LinearArgs a{};
            a.dtype = (int)ldt;
            a.x = src_ptr(st, cx, 0);
            a.w = src_ptr(st, cx, 1);
            a.m = x.dims[0]; a.k = x.dims[1]; a.n = w.dims[1];
            a.ws = cx.ws + st.scratch_off;
            a.ws_bytes = st.scratch_bytes;
            size_t i = linear_extra_pos(in);
            if (in.quant) {
                // stand-alone path of a quantised linear: the weights are dequantised into scratch and the generic
                // kernel runs over them (the decode chain and the matrix-core kernels over the codes are the fast paths)
                const size_t es = dtype_size(ldt);
                char* wsp = cx.ws + st.scratch_off;
                const size_t wbytes = align_up((size_t)a.k * a.n * es);
                auto deq = [&](size_t codes, size_t scales, void* to) {
                    if (in.quant == 1) k::dequant_w8(s, (int)ldt, (const int8_t*)src_ptr(st, cx, codes), src_ptr(st, cx, scales), to, a.k, a.n);
                    else k::dequant_w4g128(s, (int)ldt, (const uint8_t*)src_ptr(st, cx, codes), src_ptr(st, cx, scales), to, a.k, a.n);
                    ++cx.launches;
                };
                if (in.norm) {
                    const size_t gi = i + (in.has_bias ? 1 : 0) + (in.has_residual ? 1 : 0);
                    norm_into(a.x, src_ptr(st, cx, gi), wsp);
                    a.x = wsp;
                    wsp += align_up((size_t)x.count() * es);
                }
                deq(1, 2, wsp);
                a.w = wsp;
                wsp += wbytes;
                if (in.act == 2) { deq(3, 4, wsp); a.w2 = wsp; wsp += wbytes; }
                a.ws = wsp;
                a.ws_bytes = st.scratch_bytes - (size_t)(wsp - (cx.ws + st.scratch_off));
            } else if (in.act == 2) {
                a.w2 = src_ptr(st, cx, 2);
            }
            if (in.has_bias) a.bias = src_ptr(st, cx, i++);
            if (in.has_residual) a.residual = src_ptr(st, cx, i++);
            a.y = dst;
            a.act = in.act == 1 ? 1 : 0;
            a.counters = cx.counters;
            if (in.out_f32) {
                // f32 result over bf16 operands outside the fast kernels (a quantised linear with the chain switched off):
                // the generic dot stores the accumulator, the f32 residual is added by the element-wise kernel
                if (in.act != 0 || in.has_bias) fail_exec("linear: f32 result with an absorbed activation or bias");
                k::DotDesc d{};
                d.batch = 1; d.m = a.m; d.n = a.n; d.k = a.k;
                d.a_sb = 0; d.a_sm = a.k; d.a_sk = 1;
                d.b_sb = 0; d.b_sk = a.n; d.b_sn = 1;
                d.c_sb = a.m * a.n; d.c_sm = a.n;
                k::dot_generic(s, (int)ldt, a.x, a.w, dst, d, true);
                ++cx.launches;
                if (in.has_residual) { k::binary(s, 0, (int)BinaryOp::Add, dst, a.residual, dst, out.count()); ++cx.launches; }
                break;
            }
            hipEvent_t e0 = nullptr, e1 = nullptr;
            if (cx.profile) {
                GPTRS_HIP_CHECK(hipEventCreate(&e0));
                GPTRS_HIP_CHECK(hipEventCreate(&e1));
                GPTRS_HIP_CHECK(hipEventRecord(e0, s));
            }
            k::linear(s, a);
            if (cx.profile) {
                GPTRS_HIP_CHECK(hipEventRecord(e1, s));
                cx.be->prof_events.emplace_back(e0, e1);
                ++cx.be->prof_linear_calls;
                // algorithmic bytes: activations in, every weight once, result out
                cx.be->prof_linear_bytes += io_bytes + linear_weight_bytes(in, ldt, x, w);
            }
            cx.launches += (in.act == 2 && a.m > 16) ? 3 : 1;
            break;
        }
        case OpKind::FQuant: {
            const int qo = in.quant;
            if (qo == 1 || qo == 3) {
                const Spec& w = in_spec(0);
                (qo == 1 ? k::quant_w8_scales : k::quant_w4g128_scales)(s, (int)w.dtype, src_ptr(st, cx, 0), dst, w.dims[0], w.dims[1]);
            } else if (qo == 2) {
                const Spec& w = in_spec(0);
                k::quant_w8(s, (int)w.dtype, src_ptr(st, cx, 0), src_ptr(st, cx, 1), (int8_t*)dst, w.dims[0], w.dims[1]);
            } else if (qo == 4) {
                const Spec& w = in_spec(0);
                k::quant_w4g128(s, (int)w.dtype, src_ptr(st, cx, 0), src_ptr(st, cx, 1), (uint8_t*)dst, w.dims[0], w.dims[1]);
            } else if (qo == 5) {
                k::dequant_w8(s, (int)out.dtype, (const int8_t*)src_ptr(st, cx, 0), src_ptr(st, cx, 1), dst, out.dims[0], out.dims[1]);
            } else {
                k::dequant_w4g128(s, (int)out.dtype, (const uint8_t*)src_ptr(st, cx, 0), src_ptr(st, cx, 1), dst, out.dims[0], out.dims[1]);
            }
            ++cx.launches;
            break;
        }
        case OpKind::FRope: {
            const Spec& x = in_spec(0);
            k::rope_packed(s, (int)out.dtype, src_ptr(st, cx, 0), src_ptr(st, cx, 1), src_ptr(st, cx, 2), dst, x.dims[0],
                           in.n_q, in.n_kv, in.head_dim, in.rot_half);
            ++cx.launches;
            break;
        }
        case OpKind::FAttnDecode: {
            if (cx.chain && st.chain_member) break;  // executed by the launch of the run's first step
            if (cx.chain && st.chain_len > 0 && run_chain(plan, st, cx)) break;
            const Spec& ck = in_spec(1);
            k::AttnDecodeArgs a{};
            const int64_t nb = std::max<int64_t>(in.batch, 1);
            for (int64_t b = 0; b < nb; ++b) {   // caches that were not donated are copied first
                const size_t ci = attn_cache_operand(in, b), oi = attn_cache_output(b);
                void* kout = cx.ptr[st.dst[oi]];
                void* vout = cx.ptr[st.dst[oi + 1]];
                const void* kin = src_ptr(st, cx, ci);
                const void* vin = src_ptr(st, cx, ci + 1);
                if (kout != kin) { GPTRS_HIP_CHECK(hipMemcpyAsync(kout, kin, ck.bytes(), hipMemcpyDeviceToDevice, s)); ++cx.launches; }
                if (vout != vin) { GPTRS_HIP_CHECK(hipMemcpyAsync(vout, vin, ck.bytes(), hipMemcpyDeviceToDevice, s)); ++cx.launches; }
                if (b == 0) { a.k_cache = kout; a.v_cache = vout; }
                a.k_caches[b] = kout; a.v_caches[b] = vout;
            }
            a.batch = (int)in.batch;
            a.dtype = (int)out.dtype;
            a.qkv = src_ptr(st, cx, 0);
            a.update_starts = (const int32_t*)src_ptr(st, cx, 3);
            a.query_start = (const int32_t*)src_ptr(st, cx, 4);
            a.ctx = dst;
            a.n_q = in.n_q; a.n_kv = in.n_kv; a.head_dim = in.head_dim; a.capacity = ck.dims[1];
            a.scale = in.scale;
            a.ws = cx.ws + st.scratch_off;
            a.ws_bytes = st.scratch_bytes;
            if (in.rot_half > 0) { a.cos = src_ptr(st, cx, 5); a.sin = src_ptr(st, cx, 6); a.rot_half = in.rot_half; }
            cx.launches += k::attn_decode(s, a);
            break;
        }
        case OpKind::FAttnPrefill: {
            const Spec& x = in_spec(0);
            k::AttnPrefillArgs a{};
            a.dtype = (int)out.dtype;
            a.qkv = src_ptr(st, cx, 0);
            a.ctx = dst;
            a.t = x.dims[0]; a.n_q = in.n_q; a.n_kv = in.n_kv; a.head_dim = in.head_dim;
            a.scale = in.scale;
            k::attn_prefill(s, a);
            ++cx.launches;
            break;
        }
        case OpKind::FAttnConcat: {
            const Spec& x = in_spec(0);
            const Spec& ck = in_spec(1);
            k::AttnConcatArgs a{};
            a.dtype = (int)out.dtype;
            a.qkv = src_ptr(st, cx, 0);
            a.k_cache = src_ptr(st, cx, 1);
            a.v_cache = src_ptr(st, cx, 2);
            a.ctx = dst;
            a.k_all = cx.ptr[st.dst[1]];
            a.v_all = cx.ptr[st.dst[2]];
            a.t = x.dims[0]; a.cache_len = ck.dims[1]; a.n_q = in.n_q; a.n_kv = in.n_kv; a.head_dim = in.head_dim;
            a.scale = in.scale;
            k::attn_concat(s, a);
            cx.launches += 2;
            break;
        }
        default:
            fail_unimpl(in.op_name, "no kernel bound to this operation");
    }
}

}  // namespace gptrs
