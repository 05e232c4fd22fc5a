// serde-JSON -> executor IR.  Field names and enum encodings follow the derive attributes in
// crates/gpt-rs/src/backend/spec.rs (externally tagged enums, unit variants as strings).
#include "ptir.hpp"

#include <sstream>

namespace gptrs {

DType parse_dtype(const std::string& n) {
    if (n == "F32") return DType::F32;
    if (n == "Bf16") return DType::BF16;
    if (n == "Si32") return DType::SI32;
    if (n == "I1") return DType::I1;
    if (n == "Si8") return DType::SI8;
    if (n == "Ui8") return DType::UI8;
    static const char* known[] = {"Si4", "Ui4", "Si16", "Ui16", "Ui32", "Si64", "Ui64", "Fp8E4M3",
                                  "Fp8E5M2", "F16", "F64", "Cf32", "Cf64"};
    for (auto k : known)
        if (n == k) fail_spec("dtype_not_supported (dtype " + n + " unsupported by the hip backend)");
    fail_spec("unknown dtype `" + n + "`");
}

std::string Spec::str() const {
    std::ostringstream o;
    o << dtype_name(dtype) << "[";
    for (size_t i = 0; i < dims.size(); ++i) o << (i ? "," : "") << dims[i];
    o << "]";
    return o.str();
}

static std::vector<int64_t> int_list(const Json& j) {
    std::vector<int64_t> v;
    for (auto& e : j.as_array()) v.push_back(e.as_int());
    return v;
}

static std::vector<int64_t> parse_shape(const Json& shape) {
    std::vector<int64_t> dims;
    for (auto& d : shape.at("dims").as_array()) {
        if (const Json* s = d.find("Static")) {
            int64_t v = s->as_int();
            if (v < 0) fail_spec("negative dimension");
            dims.push_back(v);
        } else if (const Json* dyn = d.find("Dynamic")) {
            fail_exec("dynamic dimension " + (dyn->is_string() ? dyn->s : std::string("?")) +
                      " not supported at runtime");
        } else {
            fail_spec("malformed Dimension");
        }
    }
    return dims;
}

static Spec parse_spec(const Json& j) {
    Spec s;
    s.dtype = parse_dtype(j.at("dtype").as_string());
    s.dims = parse_shape(j.at("shape"));
    return s;
}

static Spec parse_value_type(const Json& j) {
    if (const Json* t = j.find("Tensor")) return parse_spec(*t);
    fail_exec("tuple outputs are not supported in the hip backend");
}

static int add_literal(const Json& j, Function& fn) {
    Literal lit;
    lit.spec = parse_spec(j.at("spec"));
    for (auto& b : j.at("bytes").as_array()) {
        int64_t v = b.as_int();
        if (v < 0 || v > 255) fail_spec("literal byte out of range");
        lit.bytes.push_back((uint8_t)v);
    }
    if (lit.bytes.size() != lit.spec.bytes()) fail_exec("literal byte length mismatch");
    fn.literals.push_back(std::move(lit));
    return (int)fn.literals.size() - 1;
}

template <typename E>
static E parse_enum(const Json& j, std::initializer_list<std::pair<const char*, E>> table, const char* what) {
    const std::string& s = j.as_string();
    for (auto& kv : table)
        if (s == kv.first) return kv.second;
    fail_spec(std::string("unknown ") + what + " `" + s + "`");
}

static void reject_dtype_override(const Json& attr, const char* op, DType in_dtype) {
    // cpu.rs:2118-2135: only the default accumulate-in-f32 / output-in-input-dtype policy is served.
    if (const Json* a = attr.find("accum_dtype"))
        if (!a->is_null() && a->as_string() != "F32") fail_unimpl(op, "accum_dtype override not supported");
    if (const Json* o = attr.find("out_dtype"))
        if (!o->is_null() && parse_dtype(o->as_string()) != in_dtype) fail_unimpl(op, "out_dtype not supported");
}

Instr parse_instruction(const Json& j, Function& fn) {
    Instr in;
    in.out_ids.push_back((int)j.at("id").as_int());
    in.out_specs.push_back(parse_value_type(j.at("output")));
    for (auto& od : j.at("operands").as_array()) {
        Operand o;
        if (const Json* v = od.find("Value")) o.value = (int)v->as_int();
        else if (const Json* l = od.find("Literal")) o.literal = add_literal(*l, fn);
        else fail_exec("tuple operands not supported");
        in.operands.push_back(o);
    }
    const Json& op = j.at("op");
    std::string name;
    const Json* attr = nullptr;
    if (op.is_string()) {
        name = op.s;
    } else if (op.is_object() && op.obj.size() == 1) {
        name = op.obj[0].first;
        attr = &op.obj[0].second;
    } else {
        fail_spec("malformed Operation");
    }
    in.op_name = name;
    auto need = [&](size_t n) {
        if (in.operands.size() != n)
            fail_exec(name + " expects " + std::to_string(n) + " operands, got " + std::to_string(in.operands.size()));
    };
    if (name == "Constant") {
        in.op = OpKind::Constant;
        in.literal = add_literal(*attr, fn);
    } else if (name == "ElementwiseUnary") {
        in.op = OpKind::Unary; need(1);
        in.unary = parse_enum<UnaryOp>(*attr, {{"Neg", UnaryOp::Neg}, {"Abs", UnaryOp::Abs}, {"Exp", UnaryOp::Exp},
            {"Log", UnaryOp::Log}, {"Tanh", UnaryOp::Tanh}, {"Erf", UnaryOp::Erf}, {"Rsqrt", UnaryOp::Rsqrt},
            {"Reciprocal", UnaryOp::Reciprocal}}, "unary op");
    } else if (name == "ElementwiseBinary") {
        in.op = OpKind::Binary; need(2);
        in.binary = parse_enum<BinaryOp>(*attr, {{"Add", BinaryOp::Add}, {"Sub", BinaryOp::Sub}, {"Mul", BinaryOp::Mul},
            {"Div", BinaryOp::Div}, {"Maximum", BinaryOp::Maximum}, {"Minimum", BinaryOp::Minimum}}, "binary op");
    } else if (name == "DotGeneral") {
        in.op = OpKind::Dot; need(2);
        in.a = int_list(attr->at("batch_lhs"));
        in.b = int_list(attr->at("batch_rhs"));
        in.c = int_list(attr->at("contract_lhs"));
        in.d = int_list(attr->at("contract_rhs"));
        reject_dtype_override(*attr, "dot_general", in.out_specs[0].dtype);
        if (const Json* o = attr->find("out_dtype")) in.out_f32 = !o->is_null() && in.out_specs[0].dtype == DType::F32;
    } else if (name == "Reduce") {
        in.op = OpKind::Reduce; need(1);
        in.reduce = parse_enum<ReduceKind>(attr->at("kind"), {{"Sum", ReduceKind::Sum}, {"Max", ReduceKind::Max},
            {"Min", ReduceKind::Min}}, "reduce kind");
        in.a = int_list(attr->at("axes"));
        in.keepdims = attr->at("keepdims").as_bool();
        reject_dtype_override(*attr, "reduce", in.out_specs[0].dtype);
    } else if (name == "Compare") {
        in.op = OpKind::Compare; need(2);
        in.cmp = parse_enum<CmpOp>(attr->at("op"), {{"Less", CmpOp::Less}, {"LessEqual", CmpOp::LessEqual},
            {"Equal", CmpOp::Equal}, {"GreaterEqual", CmpOp::GreaterEqual}, {"Greater", CmpOp::Greater},
            {"NotEqual", CmpOp::NotEqual}}, "comparison op");
    } else if (name == "Select") {
        in.op = OpKind::Select; need(3);
    } else if (name == "Cast") {
        in.op = OpKind::Cast; need(1);
        if (parse_dtype(attr->at("dtype").as_string()) != in.out_specs[0].dtype) fail_exec("cast output dtype mismatch");
    } else if (name == "StopGradient") {
        in.op = OpKind::StopGradient; need(1);
    } else if (name == "Reshape") {
        in.op = OpKind::Reshape; need(1);
    } else if (name == "Transpose") {
        in.op = OpKind::Transpose; need(1);
        in.a = int_list(attr->at("perm"));
    } else if (name == "BroadcastTo") {
        in.op = OpKind::BroadcastTo; need(1);
        if (parse_shape(attr->at("result_shape")) != in.out_specs[0].dims) fail_exec("broadcast_to output shape mismatch");
    } else if (name == "Slice") {
        in.op = OpKind::Slice; need(1);
        in.a = int_list(attr->at("starts"));
        in.b = int_list(attr->at("sizes"));
    } else if (name == "Concat") {
        in.op = OpKind::Concat;
        if (in.operands.empty()) fail_exec("concat expects at least one input");
        in.axis = attr->at("axis").as_int();
    } else if (name == "Iota") {
        in.op = OpKind::Iota; need(0);
        in.axis = attr->at("axis").as_int();
        if (parse_shape(attr->at("shape")) != in.out_specs[0].dims) fail_exec("iota output shape mismatch");
        if (parse_dtype(attr->at("dtype").as_string()) != in.out_specs[0].dtype) fail_exec("iota output dtype mismatch");
    } else if (name == "Take") {
        in.op = OpKind::Take; need(2);
    } else if (name == "DynamicSlice") {
        in.op = OpKind::DynamicSlice; need(2);
        in.a = int_list(attr->at("sizes"));
    } else if (name == "DynamicUpdateSlice") {
        in.op = OpKind::DynamicUpdateSlice; need(3);
        in.a = int_list(attr->at("sizes"));
    } else if (name == "CustomCall") {
        in.op = OpKind::CustomCall;
        in.target = attr->at("target").as_string();
        if (const Json* at = attr->find("attrs"))
            for (auto& kv : at->obj) in.attrs[kv.first] = kv.second;
    } else {
        // Everything the LM path never emits answers Unimplemented, as ref-cpu does (cpu.rs:326-331).
        in.op = OpKind::Unsupported;
    }
    return in;
}

Function parse_program(const char* json, size_t len) {
    Json root;
    try {
        root = JsonParser(json, len).parse();
    } catch (const JsonError& e) {
        fail_spec(e.what());
    }
    try {
        if (const Json* v = root.find("spec_version")) {
            const std::string& s = v->as_string();
            if (!s.empty() && s != "ptir.v0.4")
                fail_spec("program spec version '" + s + "' does not match expected 'ptir.v0.4'");
        }
        const std::string& entry = root.at("entry").as_string();
        const Json* fj = nullptr;
        for (auto& f : root.at("functions").as_array())
            if (f.at("name").as_string() == entry) { fj = &f; break; }
        if (!fj) fail_exec("entry function not found");
        Function fn;
        fn.name = entry;
        for (auto& p : fj->at("parameter_ids").as_array()) fn.param_ids.push_back((int)p.as_int());
        for (auto& p : fj->at("parameters").as_array()) fn.param_specs.push_back(parse_value_type(p));
        if (fn.param_ids.size() != fn.param_specs.size()) fail_spec("parameters / parameter_ids length mismatch");
        for (auto& r : fj->at("result_ids").as_array()) fn.result_ids.push_back((int)r.as_int());
        for (auto& r : fj->at("results").as_array()) fn.result_specs.push_back(parse_value_type(r));
        if (fn.result_ids.size() != fn.result_specs.size()) fail_spec("results / result_ids length mismatch");
        for (auto& ij : fj->at("body").as_array()) fn.body.push_back(parse_instruction(ij, fn));
        int mx = 0;
        for (int id : fn.param_ids) mx = std::max(mx, id);
        for (auto& in : fn.body) mx = std::max(mx, in.out_ids[0]);
        fn.max_value_id = mx;
        return fn;
    } catch (const JsonError& e) {
        fail_spec(e.what());
    }
}

}  // namespace gptrs
