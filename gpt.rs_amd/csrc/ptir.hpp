// PTIR (ptir.v0.4) program model as the executor sees it, parsed from the serde-JSON
// wire form of crates/gpt-rs/src/backend/spec.rs:644-817.
#pragma once
#include <cstdint>
#include <map>
#include <stdexcept>
#include <string>
#include <vector>

#include "json.hpp"

namespace gptrs {

// Error kinds map 1:1 onto BackendError (spec.rs:1224-1228).
enum class ErrKind { Spec = 1, Unimplemented = 2, Execution = 3 };
struct BackendError : std::runtime_error {
    ErrKind kind;
    BackendError(ErrKind k, const std::string& m) : std::runtime_error(m), kind(k) {}
};
[[noreturn]] inline void fail_spec(const std::string& m) { throw BackendError(ErrKind::Spec, m); }
[[noreturn]] inline void fail_unimpl(const std::string& op, const std::string& why) {
    throw BackendError(ErrKind::Unimplemented, op + " is not implemented: " + why);
}
[[noreturn]] inline void fail_exec(const std::string& m) {
    throw BackendError(ErrKind::Execution, "backend execution failure: " + m);
}

// Tags shared with include/gptrs_hip.h.
enum class DType : uint32_t { F32 = 0, F16 = 1, BF16 = 2, SI32 = 3, I1 = 4, SI8 = 5, UI8 = 6, Invalid = 99 };

inline size_t dtype_size(DType d) {
    switch (d) {
        case DType::F32: case DType::SI32: return 4;
        case DType::F16: case DType::BF16: return 2;
        case DType::I1: case DType::SI8: case DType::UI8: return 1;
        default: return 0;
    }
}
inline const char* dtype_name(DType d) {
    switch (d) {
        case DType::F32: return "F32"; case DType::F16: return "F16"; case DType::BF16: return "Bf16";
        case DType::SI32: return "Si32"; case DType::I1: return "I1"; case DType::SI8: return "Si8";
        case DType::UI8: return "Ui8"; default: return "?";
    }
}
inline bool dtype_is_float(DType d) { return d == DType::F32 || d == DType::BF16; }
DType parse_dtype(const std::string& name);  // throws Spec error on dtypes the backend does not execute

struct Spec {
    DType dtype = DType::F32;
    std::vector<int64_t> dims;
    int64_t count() const {
        int64_t n = 1;
        for (auto d : dims) n *= d;
        return n;
    }
    size_t bytes() const { return (size_t)count() * dtype_size(dtype); }
    int rank() const { return (int)dims.size(); }
    bool operator==(const Spec& o) const { return dtype == o.dtype && dims == o.dims; }
    bool operator!=(const Spec& o) const { return !(*this == o); }
    std::string str() const;
};

struct Literal {
    Spec spec;
    std::vector<uint8_t> bytes;
};

enum class OpKind {
    Constant, Unary, Binary, Dot, Reduce, Compare, Select, Cast, StopGradient, Reshape, Transpose,
    BroadcastTo, Slice, Concat, Iota, Take, DynamicSlice, DynamicUpdateSlice, CustomCall,
    // fused forms produced by the executor's pattern pass (never present on the wire)
    FLayerNorm, FRmsNorm, FSoftmax, FGelu, FSilu, FSwiglu, FLinear, FRope, FAttnDecode, FAttnPrefill, FAttnConcat,
    FEmbed, FQuant,
    Unsupported
};
enum class UnaryOp { Neg, Abs, Exp, Log, Tanh, Erf, Rsqrt, Reciprocal };
enum class BinaryOp { Add, Sub, Mul, Div, Maximum, Minimum };
enum class ReduceKind { Sum, Max, Min };
enum class CmpOp { Less, LessEqual, Equal, GreaterEqual, Greater, NotEqual };

struct Operand {
    int value = -1;    // SSA value id, or -1 when literal
    int literal = -1;  // index into Function::literals
};

struct Instr {
    OpKind op = OpKind::Unsupported;
    std::string op_name;             // wire name, for error messages
    std::vector<Operand> operands;
    std::vector<int> out_ids;        // one on the wire; fused ops may define several
    std::vector<Spec> out_specs;
    bool dead = false;

    // attributes (only those of `op` are meaningful)
    UnaryOp unary{};
    BinaryOp binary{};
    ReduceKind reduce{};
    CmpOp cmp{};
    std::vector<int64_t> a, b, c, d;  // dot: batch_lhs, batch_rhs, contract_lhs, contract_rhs
                                      // slice: a=starts b=sizes; transpose: a=perm; reduce: a=axes
                                      // dyn ops: a=sizes
    int64_t axis = 0;                 // concat / iota axis
    bool keepdims = true;
    int literal = -1;                 // Constant payload
    std::string target;               // CustomCall
    std::map<std::string, Json> attrs;
    // fused-op parameters
    float eps = 0.f, scale = 0.f;
    int64_t n_q = 0, n_kv = 0, head_dim = 0, rot_half = 0;
    // FAttnDecode over `batch` independent sequences in one launch (0 / 1: a single sequence): operand 0 is the
    // stacked [batch, P] projection, the caches of sequence b >= 1 follow the single-sequence operands in pairs,
    // outputs are (ctx[batch, q_proj], k_0, v_0, k_1, v_1, ...)
    int64_t batch = 0;
    int act = 0;                      // FLinear epilogue: 0 none, 1 gelu, 2 swiglu (dual weights)
    bool has_bias = false, has_residual = false;
    float fparam[4] = {0.f, 0.f, 0.f, 0.f};  // FGelu: half, divisor, one
    // DynamicUpdateSlice whose update is a view (Slice / Reshape / Transpose chain) of operand 1: the update's shape,
    // and its element strides and offset inside operand 1; empty when operand 1 is the update itself
    std::vector<int64_t> view_dims, view_strides;
    int64_t view_off = 0;
    bool mfma = false;                       // FLinear: prefill GEMM over the k-grouped weight copy
    bool tiled = false;                      // FLinear: decode GEMV over the column-tiled weight copy
    bool norm = false;                       // FLinear: RMSNorm of x fused in (last operand = gamma; eps, scale)
    bool norm_ln = false;                    // with norm: LayerNorm instead (last two operands = gamma, beta)
    // Dot / FLinear with bf16 operands whose f32 accumulator leaves as f32 (DotGeneralSpec.out_dtype = F32,
    // spec.rs:354-361); an FLinear's residual operand is then f32 too
    bool out_f32 = false;
    // FLinear with norm whose x (and gamma) are f32 while the weights are bf16: the norm runs in f32 and its result is
    // rounded to bf16 once (the fold of Cast(bf16)(rms_norm(x f32)) into the linear)
    bool x_f32 = false;
    // FLinear over weight-only quantised weights (0: none; 1: int8 per column, 2: int4 groups of 128): every
    // weight operand is then a (codes, scales) pair: (x, q, s, [q2, s2], [bias], [residual], [gamma]).
    // FQuant: 1 int8 scales, 2 int8 codes, 3 int4 scales, 4 int4 codes, 5 int8 dequantise, 6 int4 dequantise
    int quant = 0;
    bool scalar_rhs = false;                 // Binary whose rhs is a broadcast scalar literal
    float scalar_val = 0.f;
};

// FAttnDecode: operand slots of the K / V cache of sequence b, output slot of its updated K cache (V follows)
inline size_t attn_cache_operand(const Instr& in, int64_t b) { return b == 0 ? 1 : (size_t)(5 + (in.rot_half > 0 ? 2 : 0) + 2 * (b - 1)); }
inline size_t attn_cache_output(int64_t b) { return (size_t)(1 + 2 * b); }

// operand position of the SwiGLU partner's weights / of the first epilogue operand of an FLinear
inline size_t linear_w2_pos(const Instr& in) { return in.quant ? 3 : 2; }
inline size_t linear_extra_pos(const Instr& in) { return 1 + (size_t)(in.quant ? 2 : 1) * (in.act == 2 ? 2 : 1); }
// CustomCall targets of the weight-only quantisation extension (build-defined; the reference has none)
inline int quant_dot_target(const std::string& t) {
    if (t == "gpt_rs.hip.dot_w8.v1") return 1;
    if (t == "gpt_rs.hip.dot_w4g128.v1") return 2;
    return 0;
}
// CustomCall targets a front-end pass emits in place of a matched functional sequence (what a BackendPipeline's
// populate_pre pass does ahead of the parameter-only fold, crates/gpt-rs/src/backend/pipeline.rs:60-65, 89-92; the
// Triton backend's is crates/gpt-rs-backend-triton/src/optimizer/layer_norm_fusion.rs:30-97): 1 layer_norm(x, gamma,
// beta), 2 rms_norm(x, gamma); attribute "eps" (F64), reduction over the last axis
inline int norm_call_target(const std::string& t) {
    if (t == "gpt_rs.hip.layer_norm.v1") return 1;
    if (t == "gpt_rs.hip.rms_norm.v1") return 2;
    return 0;
}
inline int quant_op_target(const std::string& t) {
    if (t == "gpt_rs.hip.quantize_w8_scales.v1") return 1;
    if (t == "gpt_rs.hip.quantize_w8.v1") return 2;
    if (t == "gpt_rs.hip.quantize_w4g128_scales.v1") return 3;
    if (t == "gpt_rs.hip.quantize_w4g128.v1") return 4;
    if (t == "gpt_rs.hip.dequantize_w8.v1") return 5;
    if (t == "gpt_rs.hip.dequantize_w4g128.v1") return 6;
    return 0;
}

struct Function {
    std::string name;
    std::vector<int> param_ids;
    std::vector<Spec> param_specs;
    std::vector<int> result_ids;
    std::vector<Spec> result_specs;
    std::vector<Instr> body;
    std::vector<Literal> literals;
    int max_value_id = 0;
};

// Parses `Program` JSON and returns the entry function.  Enforces spec_version
// (spec.rs:844-856), static shapes, single tensor outputs (cpu.rs:257-266).
Function parse_program(const char* json, size_t len);
Instr parse_instruction(const Json& j, Function& fn);

}  // namespace gptrs
