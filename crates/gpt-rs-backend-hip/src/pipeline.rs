//! The backend's own optimizer hooks (`BackendPipeline`, crates/gpt-rs/src/backend/pipeline.rs:60-65).
//!
//! Not compiled in this repository's build image (no Rust toolchain there): written against the reference's sources by
//! reading.  `gpt.rs_amd/front_end.py` (`HipNormFusionPass`) is the same pass in Python, and that one is tested: CPU
//! tests check the rewritten programs, GPU tests run the models through it.
//!
//! One pass, in `populate_pre`, i.e. ahead of `ParamOnlyFoldToParamPass` (pipeline.rs:89-98): the instruction sequences
//! of `functional::layer_norm` and `functional::rms_norm` become ONE `CustomCall` each, with gamma and beta themselves
//! as operands, so the fold finds no `BroadcastTo(shape)(gamma)` to execute and replace by a derived parameter of the
//! broadcast shape.  The Triton backend solves the same problem the same way
//! (crates/gpt-rs-backend-triton/src/optimizer/{pipeline.rs:15-21, layer_norm_fusion.rs:30-97}).
//!
//! The library does not depend on this pass: a handle it produced as a pure broadcast of a vector remembers that vector,
//! and a program that takes the handle as an input is planned as if it held the `BroadcastTo` itself.  The pass is for
//! derived parameters that lose that provenance (a resolver that copies handles through the host).
use std::collections::BTreeMap;
use std::sync::Arc;

use gpt_rs::backend::index::InstId;
use gpt_rs::backend::optimizer::{FunctionPass, OptimizeContext, PassResult};
use gpt_rs::backend::pattern::OperationView;
use gpt_rs::backend::pipeline::{BackendPipeline, PipelineBuilder};
use gpt_rs::backend::rewriter::ProgramRewriter;
use gpt_rs::backend::spec::{
    CustomCallAttr, CustomCallSpec, Function, Operand, Operation, TensorLiteral, ValueId, ValueType,
};
use gpt_rs::ops::functional::normalization::{LayerNormPattern, RmsNormPattern};

use crate::HipBackend;

/// Targets the library lowers to its fused norm kernels (`include/gptrs_hip.h`, run_program).
pub const TARGET_LAYER_NORM: &str = "gpt_rs.hip.layer_norm.v1";
pub const TARGET_RMS_NORM: &str = "gpt_rs.hip.rms_norm.v1";

#[derive(Debug, Default)]
pub struct HipPipeline;

impl BackendPipeline<HipBackend> for HipPipeline {
    fn populate_pre(&self, p: &mut PipelineBuilder<HipBackend>) {
        p.pass(Arc::new(HipNormFusionPass));
    }
}

pub struct HipNormFusionPass;

/// What one match rewrites: the call's operands, its eps, the value it replaces and the sequence's instructions.
struct NormRewrite {
    target: &'static str,
    operands: Vec<ValueId>,
    eps: f32,
    output: ValueId,
    interior: Vec<InstId>,
}

impl FunctionPass<HipBackend> for HipNormFusionPass {
    fn name(&self) -> &'static str {
        "hip-norm-fusion"
    }

    fn run(&self, function: &mut Function, _cx: &mut OptimizeContext<HipBackend>) -> PassResult {
        let Ok(mut rewriter) = ProgramRewriter::new(function) else {
            return PassResult::default();
        };
        let mut result = PassResult::default();
        // roots last to first: a layer norm ends in an rms-norm-shaped tail over the centred row, and the larger
        // sequence has to claim its instructions first
        for inst in rewriter.insts_in_order().into_iter().rev() {
            if !rewriter.contains(inst) {
                continue;
            }
            let rewrite = match LayerNormPattern::extract(inst, &rewriter) {
                Some(view) => layer_norm_rewrite(&rewriter, &view),
                None => RmsNormPattern::extract(inst, &rewriter).and_then(|view| rms_norm_rewrite(&rewriter, &view)),
            };
            let Some(rw) = rewrite else { continue };
            let Some(ValueType::Tensor(out_spec)) = rewriter.type_of(rw.output).cloned() else { continue };
            let axis = out_spec.shape.dims().len() as i64 - 1;
            let mut attrs = BTreeMap::new();
            attrs.insert("eps".to_string(), CustomCallAttr::F64(f64::from(rw.eps)));
            attrs.insert("axis".to_string(), CustomCallAttr::I64(axis));
            let op = Operation::CustomCall(CustomCallSpec { target: rw.target.to_string(), attrs });
            let operands = rw.operands.iter().map(|v| Operand::Value(*v)).collect();
            let Ok((_, call)) = rewriter.insert_before(inst, op, operands, ValueType::Tensor(out_spec)) else { continue };
            rewriter.replace_all_uses(rw.output, call);
            for id in &mut rewriter.func.result_ids {
                if *id == rw.output {
                    *id = call;
                }
            }
            result.erased_insts += erase_if_dead(&mut rewriter, &rw.interior);
            result.rewrites_applied += 1;
            result.changed = true;
        }
        result.iterations = 1;
        result
    }
}

fn value_of(operand: Option<&Operand>) -> Option<ValueId> {
    match operand {
        Some(Operand::Value(v)) => Some(*v),
        _ => None,
    }
}

/// A scalar literal behind broadcasts, in the tensor's dtype (f32, or bf16 widened).
fn scalar_of(rewriter: &ProgramRewriter, operand: Option<&Operand>) -> Option<f32> {
    fn of_literal(lit: &TensorLiteral) -> Option<f32> {
        let bytes: &[u8] = lit.bytes.as_ref();
        match (lit.spec.dtype, bytes.len()) {
            (gpt_rs::backend::spec::DType::F32, 4) => Some(f32::from_le_bytes([bytes[0], bytes[1], bytes[2], bytes[3]])),
            (gpt_rs::backend::spec::DType::Bf16, 2) => Some(f32::from_bits(u32::from(u16::from_le_bytes([bytes[0], bytes[1]])) << 16)),
            _ => None,
        }
    }
    match operand? {
        Operand::Literal(lit) => of_literal(lit),
        Operand::Value(v) => {
            let inst = rewriter.inst_of(*v)?;
            match rewriter.op(inst) {
                Operation::Constant(lit) => of_literal(lit),
                Operation::BroadcastTo(_) | Operation::Reshape(_) => scalar_of(rewriter, rewriter.operands(inst).first()),
                _ => None,
            }
        }
        Operand::TupleElement { .. } => None,
    }
}

/// The side of a two-operand instruction that is not `known`.
fn other_operand<'a>(operands: &'a [Operand], known: ValueId) -> Option<&'a Operand> {
    match (value_of(operands.first()), value_of(operands.get(1))) {
        (Some(a), _) if a == known => operands.get(1),
        (_, Some(b)) if b == known => operands.first(),
        _ => None,
    }
}

fn layer_norm_rewrite(rewriter: &ProgramRewriter, view: &LayerNormPattern) -> Option<NormRewrite> {
    // the captured inputs, in the order of `capture_ptir!({ x, gamma, beta }, ..)` (normalization.rs:133)
    let (x, gamma, beta) = (view.input(0)?, view.input(1)?, view.input(2)?);
    let eps = scalar_of(rewriter, other_operand(&view.var_eps.operands, rewriter.value_of(view.var_mean.root)))?;
    if !(eps.is_finite() && eps > 0.0) || rewriter.type_of(x) != rewriter.type_of(view.output()) {
        return None;
    }
    Some(NormRewrite {
        target: TARGET_LAYER_NORM,
        operands: vec![x, gamma, beta],
        eps,
        output: view.output(),
        interior: vec![
            view.output.root, view.beta_broadcast.root, view.gamma_broadcast.root, view.normalized.root, view.inv_std_broadcast.root,
            view.inv_std.root, view.var_eps.root, view.var_mean.root, view.var_sum.root, view.centered_sq.root, view.centered.root,
            view.mean_broadcast.root, view.mean.root, view.sum.root,
        ],
    })
}

fn rms_norm_rewrite(rewriter: &ProgramRewriter, view: &RmsNormPattern) -> Option<NormRewrite> {
    let (x, gamma) = (view.input(0)?, view.input(1)?);
    // inv_rms = rsqrt(mean_square + eps): the rsqrt's operand is the Add that holds the eps literal
    let add = rewriter.inst_of(value_of(view.inv_rms.operands.first())?)?;
    let eps = scalar_of(rewriter, other_operand(rewriter.operands(add), rewriter.value_of(view.mean_square.root)))?;
    if !(eps.is_finite() && eps > 0.0) || rewriter.type_of(x) != rewriter.type_of(view.output()) {
        return None;
    }
    Some(NormRewrite {
        target: TARGET_RMS_NORM,
        operands: vec![x, gamma],
        eps,
        output: view.output(),
        interior: vec![
            view.output.root, view.gamma_broadcast.root, view.normalized.root, view.inv_rms.root, add, view.mean_square.root,
            view.sum.root, view.squared.root,
        ],
    })
}

/// Erases the listed instructions that nothing reads any more, last first, until none goes (a program that also asks
/// for the mean keeps the instructions that produce it).
fn erase_if_dead(rewriter: &mut ProgramRewriter, insts: &[InstId]) -> usize {
    let mut pending: Vec<InstId> = insts.to_vec();
    pending.sort_by_key(|i| std::cmp::Reverse(i.0));
    let mut erased = 0;
    loop {
        let before = erased;
        pending.retain(|inst| {
            if !rewriter.contains(*inst) {
                return false;
            }
            let value = rewriter.value_of(*inst);
            if !rewriter.users_of(value).is_empty() || rewriter.func.result_ids.contains(&value) {
                return true;
            }
            if rewriter.erase_inst(*inst).is_ok() {
                erased += 1;
                return false;
            }
            true
        });
        if erased == before {
            return erased;
        }
    }
}
