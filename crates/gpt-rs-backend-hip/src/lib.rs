//! `PortableBackend` over the C ABI of `libgptrs_hip.so` (`include/gptrs_hip.h`), registered as backend "hip".
//!
//! Not compiled in this repository's build image (no Rust toolchain there): written against the reference's sources
//! by reading, never type-checked.  One FFI symbol per trait method (crates/gpt-rs/src/backend/spec.rs:1288-1330);
//! error codes map onto `BackendError` as the header states.
//!
//! `pipeline()` returns the backend's own optimizer hooks (`pipeline.rs`): one pass ahead of the parameter-only fold
//! that hands the norms over as CustomCalls.  The library does its own pattern matching on the program `run_program`
//! receives, after the front end's optimizer, and it also plans a derived parameter that the fold made of
//! `BroadcastTo(shape)(gamma)` or of a bias broadcast as the broadcast it came from (the handle remembers its source
//! vector), so bias epilogues survive the fold without a pass of their own.
pub mod pipeline;

use gpt_rs::backend::pipeline::BackendPipeline;
use gpt_rs::backend::param_resolver::ParamResolver;
use gpt_rs::backend::spec::*;
use std::{
    collections::HashMap,
    ffi::CStr,
    os::raw::c_char,
    sync::{Arc, Mutex},
};

#[repr(C)]
pub struct RawBackend {
    _p: [u8; 0],
}
#[repr(C)]
pub struct RawTensor {
    _p: [u8; 0],
}
#[repr(C)]
struct Desc {
    dtype: u32,
    rank: u32,
    dims: *const i64,
}

extern "C" {
    fn gptrs_hip_create(device: i32, out: *mut *mut RawBackend) -> i32;
    fn gptrs_hip_destroy(b: *mut RawBackend);
    fn gptrs_hip_materialize(b: *mut RawBackend, d: *const Desc, bytes: *const u8, n: usize, out: *mut *mut RawTensor) -> i32;
    fn gptrs_hip_to_literal(b: *mut RawBackend, t: *const RawTensor, dst: *mut u8, cap: usize) -> i32;
    fn gptrs_hip_tensor_retain(t: *mut RawTensor);
    fn gptrs_hip_tensor_release(t: *mut RawTensor);
    fn gptrs_hip_tensor_spec(t: *const RawTensor, dtype: *mut u32, dims: *mut i64, cap: usize) -> i32;
    fn gptrs_hip_run_program_donate(
        b: *mut RawBackend, json: *const c_char, len: usize, key: u64, inputs: *const *mut RawTensor, donate: *const u8,
        n_in: usize, outputs: *mut *mut RawTensor, n_out: usize,
    ) -> i32;
    fn gptrs_hip_execute_instruction(
        b: *mut RawBackend, json: *const c_char, len: usize, inputs: *const *mut RawTensor, n_in: usize, out: *mut *mut RawTensor,
    ) -> i32;
    fn gptrs_hip_param_get(b: *mut RawBackend, id: *const u8, out: *mut *mut RawTensor) -> i32;
    fn gptrs_hip_param_set(b: *mut RawBackend, id: *const u8, t: *mut RawTensor) -> i32;
    fn gptrs_hip_supports_decode_sampling(b: *const RawBackend, temperature: f32, has_top_k: i32, has_u: i32) -> i32;
    fn gptrs_hip_sample_decode_token(
        b: *mut RawBackend, logits: *const RawTensor, temperature: f32, has_top_k: i32, has_u: i32, u: f32, token: *mut i64,
    ) -> i32;
    fn gptrs_hip_last_error() -> *const c_char;
}

/// Clone = retain, Drop = release (`TensorHandle: Clone + Send + Sync`, spec.rs:1288).
pub struct HipTensor {
    raw: *mut RawTensor,
    spec: TensorSpec,
}
unsafe impl Send for HipTensor {}
unsafe impl Sync for HipTensor {}
impl Clone for HipTensor {
    fn clone(&self) -> Self {
        unsafe { gptrs_hip_tensor_retain(self.raw) };
        Self { raw: self.raw, spec: self.spec.clone() }
    }
}
impl Drop for HipTensor {
    fn drop(&mut self) {
        unsafe { gptrs_hip_tensor_release(self.raw) }
    }
}

fn check(code: i32) -> BackendResult<()> {
    if code == 0 {
        return Ok(());
    }
    let msg = unsafe { CStr::from_ptr(gptrs_hip_last_error()) }.to_string_lossy().into_owned();
    Err(match code {
        1 => BackendError::spec(SpecErrorCode::InvalidAttributeValue, msg), // SpecViolation
        2 => BackendError::unimplemented("hip", msg),                        // Unimplemented
        _ => BackendError::execution(msg),                                   // Execution
    })
}

/// dtype tags of `include/gptrs_hip.h`
fn dtype_tag(d: DType) -> BackendResult<u32> {
    Ok(match d {
        DType::F32 => 0,
        DType::F16 => 1,
        DType::Bf16 => 2,
        DType::Si32 => 3,
        DType::I1 => 4,
        DType::Si8 => 5,
        DType::Ui8 => 6,
        other => return Err(BackendError::unimplemented("hip", format!("dtype {other:?}"))),
    })
}

fn dtype_of_tag(tag: u32) -> BackendResult<DType> {
    Ok(match tag {
        0 => DType::F32,
        1 => DType::F16,
        2 => DType::Bf16,
        3 => DType::Si32,
        4 => DType::I1,
        5 => DType::Si8,
        6 => DType::Ui8,
        other => return Err(BackendError::execution(format!("unknown dtype tag {other}"))),
    })
}

/// dtype and dims of a handle, as the library holds them (`gptrs_hip_tensor_spec`).
fn spec_of_raw(raw: *const RawTensor) -> BackendResult<TensorSpec> {
    let mut tag = 0u32;
    let mut dims = [0i64; 8];
    let rank = unsafe { gptrs_hip_tensor_spec(raw, &mut tag, dims.as_mut_ptr(), dims.len()) };
    if rank < 0 || rank as usize > dims.len() {
        return Err(BackendError::execution("tensor handle without a spec"));
    }
    let dims: Vec<Dimension> = dims[..rank as usize].iter().map(|&d| Dimension::Static(d as usize)).collect();
    Ok(TensorSpec::new(dtype_of_tag(tag)?, Shape::new(dims)))
}

/// The parameter memo of the library, keyed by the 16 little-endian bytes of the reference's stable id (u128).
pub struct HipParams {
    raw: *mut RawBackend,
}
unsafe impl Send for HipParams {}
unsafe impl Sync for HipParams {}
impl ParamResolver for HipParams {
    type Handle = HipTensor;
    fn get(&self, stable_id: u128) -> Option<HipTensor> {
        let mut out = std::ptr::null_mut();
        let id = stable_id.to_le_bytes();
        if unsafe { gptrs_hip_param_get(self.raw, id.as_ptr(), &mut out) } != 0 || out.is_null() {
            return None;
        }
        match spec_of_raw(out) {
            Ok(spec) => Some(HipTensor { raw: out, spec }),
            Err(_) => {
                unsafe { gptrs_hip_tensor_release(out) };
                None
            }
        }
    }
    fn set(&self, stable_id: u128, handle: HipTensor) {
        let id = stable_id.to_le_bytes();
        unsafe { gptrs_hip_param_set(self.raw, id.as_ptr(), handle.raw) };
    }
}

/// The wire form of a program and the key the library caches its plan under.
struct WireProgram {
    json: String,
    key: u64,
}

pub struct HipBackend {
    raw: *mut RawBackend,
    params: Arc<HipParams>,
    /// serde-JSON text per program, found again by the FNV-1a hash of the program's bincode bytes.  `run_program`
    /// receives `&Program` and nothing else (the arena's `PlanKey.hash`, ops/graph/arena.rs:993, does not cross the
    /// trait), and a decode step's program is a few thousand instructions: serialising it to JSON and hashing a
    /// megabyte of text on every step would cost more than the step.  bincode is several times cheaper and exact.
    wire: Mutex<HashMap<u64, Arc<WireProgram>>>,
}
unsafe impl Send for HipBackend {}
unsafe impl Sync for HipBackend {}

impl HipBackend {
    pub fn new(device: i32) -> BackendResult<Self> {
        let mut raw = std::ptr::null_mut();
        check(unsafe { gptrs_hip_create(device, &mut raw) })?;
        Ok(Self { raw, params: Arc::new(HipParams { raw }), wire: Mutex::new(HashMap::new()) })
    }

    fn wire_form(&self, program: &Program) -> BackendResult<Arc<WireProgram>> {
        let bytes = program.to_bincode_bytes().map_err(|e| BackendError::execution(e.to_string()))?; // spec.rs:808-810
        let key = bytes.iter().fold(0xcbf29ce484222325u64, |h, b| (h ^ *b as u64).wrapping_mul(0x100000001b3)) | 1;
        let mut cache = self.wire.lock().expect("wire cache poisoned");
        if let Some(hit) = cache.get(&key) {
            return Ok(hit.clone());
        }
        if cache.len() >= 64 {
            cache.clear(); // the arena keeps 64 programs (ops/graph/plan.rs:20-29); the library's plans have their own LRU
        }
        let json = program.to_json_string().map_err(|e| BackendError::execution(e.to_string()))?; // spec.rs:799-801
        let entry = Arc::new(WireProgram { json, key });
        cache.insert(key, entry.clone());
        Ok(entry)
    }
}
impl Drop for HipBackend {
    fn drop(&mut self) {
        unsafe { gptrs_hip_destroy(self.raw) }
    }
}

impl PortableBackend for HipBackend {
    type TensorHandle = HipTensor;

    fn backend_name(&self) -> &str {
        "hip"
    }

    fn pipeline(&self) -> Option<Arc<dyn BackendPipeline<Self>>> {
        Some(Arc::new(pipeline::HipPipeline))
    }

    fn param_resolver(&self) -> Option<Arc<dyn ParamResolver<Handle = HipTensor>>> {
        Some(self.params.clone())
    }

    fn materialize(&self, init: TensorInit) -> BackendResult<HipTensor> {
        let (spec, bytes) = match &init {
            TensorInit::Literal(l) => (l.spec.clone(), Some(&l.bytes)),
            TensorInit::Zeroed(s) => (s.clone(), None),
        };
        let dims: Vec<i64> = spec
            .shape
            .static_dims()
            .ok_or_else(|| BackendError::execution("dynamic dims"))?
            .iter()
            .map(|&d| d as i64)
            .collect();
        let d = Desc { dtype: dtype_tag(spec.dtype)?, rank: dims.len() as u32, dims: dims.as_ptr() };
        let mut out = std::ptr::null_mut();
        let (p, n) = bytes.map(|b| (b.as_ptr(), b.len())).unwrap_or((std::ptr::null(), 0));
        check(unsafe { gptrs_hip_materialize(self.raw, &d, p, n, &mut out) })?;
        Ok(HipTensor { raw: out, spec })
    }

    fn to_literal(&self, t: &HipTensor) -> BackendResult<TensorLiteral> {
        let mut buf = vec![0u8; t.spec.byte_len().unwrap()];
        check(unsafe { gptrs_hip_to_literal(self.raw, t.raw, buf.as_mut_ptr(), buf.len()) })?;
        Ok(TensorLiteral::new(t.spec.clone(), buf.into()))
    }

    fn run_program(&self, program: &Program, inputs: &[HipTensor]) -> BackendResult<Vec<HipTensor>> {
        let wire = self.wire_form(program)?;
        let f = program
            .functions
            .iter()
            .find(|f| f.name == program.entry)
            .ok_or_else(|| BackendError::execution("entry function not found"))?;
        let raw: Vec<*mut RawTensor> = inputs.iter().map(|t| t.raw).collect();
        let mut outs = vec![std::ptr::null_mut(); f.result_ids.len()];
        // donate = NULL: the arena still holds clones of every input, so nothing may be consumed here
        check(unsafe {
            gptrs_hip_run_program_donate(
                self.raw, wire.json.as_ptr() as _, wire.json.len(), wire.key, raw.as_ptr(), std::ptr::null(), raw.len(),
                outs.as_mut_ptr(), outs.len(),
            )
        })?;
        let mut handles = Vec::with_capacity(outs.len());
        for (raw, ty) in outs.into_iter().zip(&f.results) {
            // (a handle is owned from here on: an error below releases the ones already wrapped through Drop)
            handles.push(HipTensor { raw, spec: tensor_spec_of(ty).or_else(|_| spec_of_raw(raw))? });
        }
        Ok(handles)
    }

    fn execute_instruction(&self, instruction: &Instruction, inputs: &[HipTensor]) -> BackendResult<Vec<HipTensor>> {
        let json = serde_json::to_string(instruction).map_err(|e| BackendError::execution(e.to_string()))?;
        let raw: Vec<*mut RawTensor> = inputs.iter().map(|t| t.raw).collect();
        let mut out = std::ptr::null_mut();
        check(unsafe { gptrs_hip_execute_instruction(self.raw, json.as_ptr() as _, json.len(), raw.as_ptr(), raw.len(), &mut out) })?;
        Ok(vec![HipTensor { raw: out, spec: spec_of_raw(out)? }])
    }

    fn supports_decode_sampling(&self, r: DecodeSampleRequest) -> bool {
        unsafe { gptrs_hip_supports_decode_sampling(self.raw, r.temperature, r.top_k.is_some() as i32, r.random_u.is_some() as i32) != 0 }
    }

    fn sample_decode_token(&self, logits: &HipTensor, _: &TensorSpec, r: DecodeSampleRequest) -> BackendResult<Option<usize>> {
        let mut tok = -1i64;
        check(unsafe {
            gptrs_hip_sample_decode_token(
                self.raw, logits.raw, r.temperature, r.top_k.is_some() as i32, r.random_u.is_some() as i32, r.random_u.unwrap_or(0.0), &mut tok,
            )
        })?;
        Ok(if tok < 0 { None } else { Some(tok as usize) })
    }
}

fn tensor_spec_of(ty: &ValueType) -> BackendResult<TensorSpec> {
    match ty {
        ValueType::Tensor(spec) => Ok(spec.clone()),
        _ => Err(BackendError::execution("the hip backend produces tensor values only")),
    }
}

/// Registers the backend under "hip" (crates/gpt-rs-backend-ref-cpu/src/lib.rs:13-23 does the same for "cpu").
pub fn register_hip_backend() {
    gpt_rs::backend::registry::register_portable_backend("hip", || HipBackend::new(0).expect("no HIP device"));
}

// Auto-register on library load, through the re-export as the reference's backends do
#[gpt_rs::linkme::distributed_slice(gpt_rs::backend::registry::BACKEND_REGISTRARS)]
static REGISTER_HIP_BACKEND: fn() = register_hip_backend;
