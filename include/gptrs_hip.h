/*
 * gptrs_hip.h -- C ABI of the MI355X (gfx950) PTIR backend, libgptrs_hip.so.
 *
 * One entry point per method of the reference's `PortableBackend` trait
 * (crates/gpt-rs/src/backend/spec.rs:1287-1349) plus the `ParamResolver` pair
 * (crates/gpt-rs/src/backend/param_resolver.rs:11-50).  A Rust shim crate binds these
 * with `extern "C"` and implements the trait over them; nothing here exposes torch,
 * HIP or C++ types.
 *
 * Return codes select the `BackendError` variant (spec.rs:1224-1228):
 *   0 ok, 1 SpecViolation, 2 Unimplemented, 3 Execution.
 * `gptrs_hip_last_error` returns the message of the calling thread's last failure.
 *
 * Threading: every entry point may be called from any thread (`Send + Sync`,
 * spec.rs:1287); calls on one backend are serialised internally.
 */
#ifndef GPTRS_HIP_H
#define GPTRS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GPTRS_HIP_OK 0
#define GPTRS_HIP_ERR_SPEC 1
#define GPTRS_HIP_ERR_UNIMPLEMENTED 2
#define GPTRS_HIP_ERR_EXECUTION 3

/* dtype tags: 0..4 are the reference C backend's PtirTensor tags
 * (crates/gpt-rs-backend-c/src/codegen/mod.rs:71-75); 5..7 extend them. */
#define GPTRS_HIP_F32 0u
#define GPTRS_HIP_F16 1u
#define GPTRS_HIP_BF16 2u
#define GPTRS_HIP_SI32 3u
#define GPTRS_HIP_I1 4u
#define GPTRS_HIP_SI8 5u
#define GPTRS_HIP_UI8 6u

typedef struct gptrs_hip_backend gptrs_hip_backend;
typedef struct gptrs_hip_tensor gptrs_hip_tensor;

/* Same field order as the reference C backend's PtirTensor minus the data pointer
 * (crates/gpt-rs-backend-c/src/codegen/mod.rs:64-69): a TensorSpec (spec.rs:210-232)
 * with static dims. */
typedef struct {
    uint32_t dtype;
    uint32_t rank;
    const int64_t* dims;
} gptrs_hip_tensor_desc;

/* Backend construction: the registry constructor `register_portable_backend("hip", ctor)`
 * (crates/gpt-rs/src/backend/registry.rs:246-260) calls this once per backend instance. */
int gptrs_hip_create(int device, gptrs_hip_backend** out);
void gptrs_hip_destroy(gptrs_hip_backend* b);

/* PortableBackend::backend_name (spec.rs:1291): returns "hip". */
const char* gptrs_hip_backend_name(const gptrs_hip_backend* b);

/* PortableBackend::materialize (spec.rs:1311): TensorInit::Literal when host_bytes is
 * non-NULL (row-major little-endian, nbytes must equal the spec's byte length),
 * TensorInit::Zeroed when it is NULL. */
int gptrs_hip_materialize(gptrs_hip_backend* b, const gptrs_hip_tensor_desc* desc,
                          const void* host_bytes, size_t nbytes, gptrs_hip_tensor** out);

/* PortableBackend::to_literal (spec.rs:1314): copies the tensor to host memory.
 * cap must be at least the tensor's byte length. */
int gptrs_hip_to_literal(gptrs_hip_backend* b, const gptrs_hip_tensor* t, void* host_dst, size_t cap);

/* TensorHandle: Clone / Drop (spec.rs:1288).  Handles are reference counted. */
void gptrs_hip_tensor_retain(gptrs_hip_tensor* t);
void gptrs_hip_tensor_release(gptrs_hip_tensor* t);

/* Spec of a handle (what `DeviceTensor::tensor_spec` carries on the Rust side).
 * dims_out receives up to dims_cap extents; returns the rank, or -1 on a NULL handle. */
int gptrs_hip_tensor_spec(const gptrs_hip_tensor* t, uint32_t* dtype_out, int64_t* dims_out, size_t dims_cap);

/* PortableBackend::run_program (spec.rs:1324; call site ops/graph/arena.rs:1014).
 * program_json: serde-JSON text of `Program` (spec.rs:799-807).  program_key: any
 * non-zero 64-bit key that identifies this text (PlanKey.hash, arena.rs:993); the parsed,
 * fused and planned form is cached under it.  0 disables the cache.
 * inputs follow `function.parameter_ids`, outputs follow `function.result_ids`;
 * n_out must equal the number of results.  Each output is a new handle owned by the
 * caller.  Inputs are left unchanged. */
int gptrs_hip_run_program(gptrs_hip_backend* b, const char* program_json, size_t json_len,
                          uint64_t program_key, gptrs_hip_tensor* const* inputs, size_t n_in,
                          gptrs_hip_tensor** outputs, size_t n_out);

/* run_program with buffer donation: donate[i] != 0 tells the backend that the caller
 * drops input i right after the call (what the models do with the previous step's KV
 * caches, crates/gpt-rs/src/model/gpt.rs:738-747), so a DynamicUpdateSlice of it may
 * write in place.  A donated handle is consumed: it stays releasable, but reading it
 * afterwards is an Execution error.  donate may be NULL (no donation). */
int gptrs_hip_run_program_donate(gptrs_hip_backend* b, const char* program_json, size_t json_len,
                                 uint64_t program_key, gptrs_hip_tensor* const* inputs,
                                 const uint8_t* donate, size_t n_in,
                                 gptrs_hip_tensor** outputs, size_t n_out);

/* PortableBackend::execute_instruction (spec.rs:1317): one Instruction as JSON, operands
 * positional (literal operands are taken from the JSON). */
int gptrs_hip_execute_instruction(gptrs_hip_backend* b, const char* instruction_json, size_t json_len,
                                  gptrs_hip_tensor* const* inputs, size_t n_in, gptrs_hip_tensor** output);

/* ParamResolver::get / set (param_resolver.rs:11-19): stable u128 id, little-endian.
 * get stores NULL in *out when the id is unknown; a returned handle is retained for
 * the caller.  set retains the handle for the memo. */
int gptrs_hip_param_get(gptrs_hip_backend* b, const uint8_t id[16], gptrs_hip_tensor** out);
int gptrs_hip_param_set(gptrs_hip_backend* b, const uint8_t id[16], gptrs_hip_tensor* t);

/* PortableBackend::supports_decode_sampling (spec.rs:1333): 1 for greedy
 * (temperature <= 0) and for temperature sampling with a caller-supplied uniform
 * random_u and no top_k; 0 otherwise. */
int gptrs_hip_supports_decode_sampling(const gptrs_hip_backend* b, float temperature, int has_top_k,
                                       int has_random_u);

/* PortableBackend::sample_decode_token (spec.rs:1341): samples from the LAST row of a
 * [rows, vocab] (or [vocab]) logits tensor on the device; 8 bytes cross PCIe.
 * Greedy ties go to the smallest index (docs/backend.md:270).  *token_out = -1 means
 * Ok(None): the request is not served here and the host sampler must run. */
int gptrs_hip_sample_decode_token(gptrs_hip_backend* b, const gptrs_hip_tensor* logits, float temperature,
                                  int has_top_k, int has_random_u, float random_u, int64_t* token_out);

/* sample_decode_token in two halves, for a decode loop that queues step t+1 before it has seen token t.  No
 * counterpart in the reference: its loop (crates/gpt-rs/src/inference/generate.rs:96-140) waits for each token
 * before it builds the next step, which leaves the device idle for a host round trip per token.
 * _begin queues the sampling of the last logits row (same rules and same kernels as sample_decode_token) and a copy
 * of the token into pinned host memory, and returns at once with *ticket_out >= 0, or -1 for Ok(None).
 * The sampled token also stays on the device: gptrs_hip_decode_token_tensor returns a new handle (si32[1]) over the
 * sampling output, valid as the token-id input of the next step's program; it is overwritten by the next _begin or
 * sample_decode_token, in stream order, so a program queued before that still reads its own token.
 * _wait blocks until the token of `ticket` has arrived (not until the queue is empty) and reports device errors
 * raised up to that point.  At most 32 tickets can be outstanding; older ones expire. */
int gptrs_hip_sample_decode_token_begin(gptrs_hip_backend* b, const gptrs_hip_tensor* logits, float temperature,
                                        int has_top_k, int has_random_u, float random_u, int64_t* ticket_out);
int gptrs_hip_sample_decode_token_wait(gptrs_hip_backend* b, int64_t ticket, int64_t* token_out);
int gptrs_hip_decode_token_tensor(gptrs_hip_backend* b, gptrs_hip_tensor** out);

/* The pipelined halves for a BATCH of independent sequences decoded together (the reference has no batch dimension,
 * crates/gpt-rs/src/ops/functional/attention.rs:189-203, so this has no counterpart there either): _rows_begin queues
 * the greedy token (largest logit, smallest index on ties, docs/backend.md:270) of EVERY row of logits [rows <= 64,
 * vocab] and returns a ticket; the tokens stay on the device in the si32[rows] tensor of gptrs_hip_decode_rows_tensor,
 * which the next step's program takes as its token-id input; _rows_wait copies the ticket's tokens out (n must equal
 * the rows the ticket was drawn for).  Tickets share the ring of sample_decode_token_begin. */
int gptrs_hip_sample_decode_rows_begin(gptrs_hip_backend* b, const gptrs_hip_tensor* logits, int64_t* ticket_out);
int gptrs_hip_sample_decode_rows_wait(gptrs_hip_backend* b, int64_t ticket, int32_t* tokens_out, size_t n);
int gptrs_hip_decode_rows_tensor(gptrs_hip_backend* b, int64_t rows, gptrs_hip_tensor** out);

/* No counterpart in the reference.  For callers that cannot allocate device memory: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  The device half of gptrs_hip_sample_decode_rows_begin with the output
 * handed in: queues, on the backend's stream, the greedy token (largest logit, smallest index on ties) of every row of
 * logits [rows, vocab] (f32 or bf16) into tokens_out, a si32 tensor of `rows` elements that the caller materialised
 * beforehand, and returns without waiting.  It launches two kernels and calls no hipMalloc / hipFree or any other
 * allocating routine; the per-block partial maxima go to a fixed 32 KiB array that the library holds on each GPU for
 * the life of the process (4096 partials), which limits rows to 64; more rows are rejected with an Execution error and
 * nothing is launched.  All calls on one GPU share that array: calls that overlap in time on one GPU (two backends on
 * one device) race.  Read the tokens with gptrs_hip_to_literal or feed tokens_out to the next program. */
int gptrs_hip_sample_decode_rows_into(gptrs_hip_backend* b, const gptrs_hip_tensor* logits, gptrs_hip_tensor* tokens_out);

/* No counterpart in the reference (a diagnostic; it touches no device and needs no backend).  Parses a program, runs the
 * backend's fusion pass on it as gptrs_hip_run_program would, and writes one line per instruction that remains, its name
 * followed for a fused linear layer by what it absorbed ("+rms_norm", "+layer_norm", "+bias", "+gelu", "+swiglu",
 * "+residual") and the kernel family it was assigned ("[stream]" the weight-streaming decode kernels, "[gemm]" the
 * matrix-core GEMM, "[generic]").  bcast_len (n_in entries, or NULL) says which inputs would arrive as handles this
 * backend produced by broadcasting a vector of that many values along leading axes (0: an ordinary input): the
 * reference's optimizer folds `BroadcastTo(shape)(gamma)` and bias broadcasts into such derived parameters before
 * run_program (crates/gpt-rs/src/backend/passes/param_only_fold_to_param.rs:24-160), and the planner reads them as the
 * broadcast they came from.  The text is truncated to cap - 1 bytes and terminated; *needed receives the size of the
 * whole text with its terminator. */
int gptrs_hip_fusion_report(const char* program_json, size_t json_len, const int64_t* bcast_len, size_t n_in, char* out, size_t cap,
                            size_t* needed);

/* Message of the calling thread's most recent non-zero return (BackendError Display). */
const char* gptrs_hip_last_error(void);

/* Blocks until all work queued by this backend has finished (used around timed regions;
 * to_literal and sample_decode_token synchronise by themselves). */
int gptrs_hip_synchronize(gptrs_hip_backend* b);

/* Execution options: name in {"fusion", "profile", "graphs", "chain", "chain_f32_min_kb", "chain_stall_phase", "gemm_lds_direct",
 * "drop_derived_weights", "evict_packed_weights"};
 * value 0/1 unless stated.
 * "fusion" = rewrite matched functional sequences to fused kernels (on by default; off = one generic kernel per
 * instruction, the reference harness's "optimizer off" leg,
 * crates/gpt-rs-backend-tests/src/torch_parity/harness.rs:494-511).  "profile" = bracket every
 * linear-layer launch with HIP events on the execution stream (the per-op ns/calls counters the
 * reference C backend exports, crates/gpt-rs-backend-c/src/lib.rs:587-671); setting it resets
 * the linear_* counters.  "graphs" (default 1) = replay a cached program that runs again over the
 * same buffer addresses as a recorded HIP graph, one launch per program instead of one per kernel
 * (no counterpart in the reference: its backends launch op by op).
 * "chain" (default 1) = run a decode step's linear layers and attention as one persistent launch (no counterpart either).
 * "chain_f32_min_kb" (default 4096) = f32 linear layers (with LayerNorm, bias, GELU, residual and f32 decode attention) join a
 * persistent launch only when they stream at least this many KiB of weights each on average: a phase of the launch costs
 * what a small stand-alone kernel costs; GPT-2 small (7 MB per layer) runs on the launch (its steady decode step takes the
 * same time either way, a whole generate call of 64 tokens is 7 % shorter), narrower f32 models on stand-alone kernels; 0 = always.
 * "gemm_lds_direct" (default 1) = unquantised bf16 linear layers of more than 16 rows run on the GEMM whose tiles go from
 * memory to LDS without passing through registers; 0 = on the register-staged GEMM that serves f32 and quantised weights
 * (the two sum in different orders: results agree to bf16 rounding, not bit for bit).
 * "chain_stall_phase" (default -1; a test hook) = value >= 1: the next persistent launch expects, at that phase's grid
 * barrier, one arrival more than its workgroups can deliver, so that its bounded wait gives up: the call that next
 * synchronises reports an Execution error and the option returns to -1.
 * "drop_derived_weights" = 1 (an action, not a state): frees the re-ordered weight copies that the kernels built at
 * first use (and the recorded graphs that point at them) and returns cached device blocks to the driver; copies still
 * needed are rebuilt by the next call that uses them.  For a caller that has finished with a kernel family, e.g. the
 * prefill copies of a server that only decodes from then on ("bytes_allocated" shows the effect).
 * "evict_packed_weights" (default 1; no counterpart in the reference, whose backends read a weight where it was
 * materialised): an unquantised bf16 matrix that a program only ever uses as the weight of linear layers, and of which
 * the persistent decode launch has built its copy, frees its row-major storage after that program ran (the copy is a
 * permutation of the matrix).  It is rebuilt from the copy, bit for bit, whenever something reads the tensor itself:
 * to_literal, a program that uses it in any other way, a kernel family that has no copy of it yet, or
 * "drop_derived_weights".  With prefill and decode copies both built, a model then holds its linear weights twice instead
 * of three times. */
int gptrs_hip_set_option(gptrs_hip_backend* b, const char* name, int64_t value);

/* Counters since creation (the reference's cache_event / WorkStats fields,
 * crates/gpt-rs/src/ops/graph/arena.rs:1201-1243): name in {"kernel_launches",
 * "programs_compiled", "program_cache_hits", "fused_ops", "bytes_allocated",
 * "inplace_updates", "last_program_launches", "derived_weights_built" (column-tiled weight copies
 * made for the decode GEMV), "graph_launches", "graphs_built", "graphs_refused" (recorded graphs with a node outside
 * what a queue accepts: such a step runs launch by launch), "chain_launches", "chain_phases", "weights_evicted" / "weights_restored"
 * (row-major weight storage freed in favour of the decode copy / rebuilt from it), and with the "profile" option "linear_time_ns",
 * "linear_calls", "linear_bytes" (these three synchronise)}.  Unknown names return -1. */
int64_t gptrs_hip_counter(const gptrs_hip_backend* b, const char* name);

#ifdef __cplusplus
}
#endif
#endif /* GPTRS_HIP_H */
