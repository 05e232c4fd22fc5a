// Host runtime of the hip PTIR backend: device buffers, tensor handles, the stable-id parameter
// memo and compiled-program (plan) cache.  One Backend owns one device and one HIP stream; every
// kernel, copy and readback is ordered on that stream.
#pragma once
#include <hip/hip_runtime.h>

#include <array>
#include <atomic>
#include <list>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "kernels.hpp"
#include "ptir.hpp"

namespace gptrs {

#define GPTRS_HIP_CHECK(expr)                                                                      \
    do {                                                                                           \
        hipError_t e_ = (expr);                                                                    \
        if (e_ != hipSuccess)                                                                      \
            ::gptrs::fail_exec(std::string(#expr) + " failed: " + hipGetErrorString(e_));          \
    } while (0)

class Backend;
struct ExecCtx;

// Size-bucketed cache of device allocations (the reference's Triton backend keeps the same kind
// of cache, crates/gpt-rs-backend-triton/src/device.rs:727-751).  Blocks are only ever used on the
// backend's single stream, so a freed block may be handed out again immediately.
class DevicePool {
  public:
    void* alloc(size_t bytes, size_t* cap_out);
    void release(void* p, size_t cap);
    void trim();  // return every cached block to the driver
    size_t bytes_allocated = 0;

  private:
    static size_t bucket(size_t n);
    std::unordered_map<size_t, std::vector<void*>> free_;
};

struct Buffer {
    void* ptr = nullptr;
    size_t cap = 0;
    Backend* owner = nullptr;
    uint64_t id = 0;  // identity of the CONTENTS: fresh per allocation, bumped when updated in place
    bool has_derived = false;  // some derived weight layout was built from this buffer
    // A bf16 weight whose decode-chain copy exists holds the same values twice.  Once no kernel of the programs that
    // use it reads the row-major form, that form is given back (`evicted`: ptr is null, `cap` still says how much to
    // allocate) and Backend::ensure_resident rebuilds it from the copy named by `chain_key` when something asks.
    bool evicted = false;
    std::array<uint64_t, 3> chain_key{{0, 0, 0}};   // key of the chain copy built from this buffer ({0,0,0}: none)
    ~Buffer();
};
using BufferP = std::shared_ptr<Buffer>;
struct Plan;

}  // namespace gptrs

// The opaque handle type of include/gptrs_hip.h.
struct gptrs_hip_tensor {
    std::atomic<int> refs{1};
    gptrs::Spec spec;
    mutable gptrs::BufferP buf;
    bool consumed = false;  // donated to a run_program call
    // A tensor this backend produced as a pure broadcast of a vector x[n] along leading axes (what the reference's
    // ParamOnlyFoldToParamPass makes of `BroadcastTo(in)(gamma)` and of a bias broadcast,
    // crates/gpt-rs/src/backend/passes/param_only_fold_to_param.rs:24-160): `bcast_src` is that vector (retained).  A
    // program that takes such a tensor as an input is planned as if it held the BroadcastTo instruction itself, so the
    // norm / bias patterns match and their kernels read the n values.  Until something reads the broadcast data
    // itself, the handle has no buffer: `lazy_plan` run on `lazy_input` produces it (Backend::realize).
    gptrs_hip_tensor* bcast_src = nullptr;
    mutable std::shared_ptr<gptrs::Plan> lazy_plan;
    mutable gptrs_hip_tensor* lazy_input = nullptr;
    gptrs::Backend* backend = nullptr;   // set on handles without a buffer (the owner of a buffer is found through it)
    void* data() const { return buf ? buf->ptr : nullptr; }
};

namespace gptrs {

// ---- compiled program -------------------------------------------------------------------
enum class Storage { Input, Temp, Output, Const, InPlace };

struct ValueInfo {
    Spec spec;
    int root = -1;  // value whose storage this one aliases (itself when it owns storage)
    bool defined = false;
};

struct RootStorage {
    Storage kind = Storage::Temp;
    int index = 0;       // Input: input position; Output: output-buffer index; InPlace: input position
    size_t offset = 0;   // Temp: byte offset in the workspace; Const: offset in the const block
    size_t bytes = 0;
};

struct Step {
    Instr in;                      // attributes (operands resolved below)
    std::vector<int> src;          // operand value ids (-1 for literal operands)
    std::vector<size_t> src_const; // const-block offset for literal operands
    std::vector<int> dst;          // output value ids
    // precomputed launch descriptors
    std::vector<k::CopyDesc> copies;  // strided copies (one per concat operand, etc.)
    int elem_size = 0;
    k::DotDesc dot{};
    int64_t outer = 0, axis_len = 0, inner = 0;
    float scalar = 0.f;
    bool rhs_scalar = false;
    size_t scratch_off = 0, scratch_bytes = 0;  // per-step scratch inside the workspace
    bool copy_base = false;        // DynamicUpdateSlice / FAttnDecode: copy base -> out first
    bool lhs_pack = false, rhs_pack = false;    // Dot: operands repacked into scratch first
    int tiled_w_input = -1, tiled_w2_input = -1;  // FLinear over column-tiled weights: input positions of W, W2
    int tiled_s_input = -1, tiled_s2_input = -1;  // ... and of their scale tensors when the weights are quantised
    // Run of consecutive decode linears executed by ONE persistent launch (kernels_chain.hip): the
    // first step of the run carries its length, the others are marked as members.
    int chain_len = 0;
    bool chain_member = false;
    k::CopyDesc pack_l{}, pack_r{};
    size_t pack_l_off = 0, pack_r_off = 0;
};

// A captured replay of one plan for one set of buffer addresses.
struct PlanGraph {
    std::vector<uint64_t> key;  // input/output addresses + content ids of the weights read through derived copies
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    uint64_t last_use = 0;
    int64_t launches = 0;
    std::vector<const void*> tables;  // device tables of phases that its persistent launches read
};

struct Plan {
    ~Plan();
    bool cacheable = false;                 // lives in the plan LRU (program_key != 0)
    std::vector<PlanGraph> graphs;
    std::vector<uint64_t> seen_keys;        // hashes of address sets executed eagerly so far (ring)
    int64_t graph_builds = 0, graph_hits = 0, runs = 0;
    uint64_t graph_clock = 0;
    Function fn;
    std::vector<ValueInfo> values;          // indexed by value id
    std::vector<RootStorage> storage;       // indexed by value id (meaningful for roots)
    std::vector<Step> steps;
    std::vector<int> out_buffer_of_result;  // result position -> output buffer index (or -1: aliases an input)
    std::vector<int> result_input_alias;    // result position -> input position it aliases, or -1
    std::vector<size_t> out_buffer_bytes;
    std::vector<int> out_buffer_inplace_input;  // output buffer index -> donated input position or -1
    // Inputs that arrived tagged as broadcasts of a vector: `ext_inputs[j]` is the position of the caller's input whose
    // source vector is fed as input n_user_inputs + j (the function was rewritten to read BroadcastTo(vector) in place
    // of that input before the fusion pass ran).
    size_t n_user_inputs = 0;
    std::vector<int> ext_inputs;
    std::vector<bool> input_read;           // per (extended) input: some step or result reads its storage
    // per (extended) input: every use is the weight of an unquantised linear that runs on a derived layout, so no
    // kernel of this plan reads the input's own storage
    std::vector<bool> input_weight_only;
    // result position -> the caller's input it is a pure broadcast of along leading axes (or -1)
    std::vector<int> result_bcast_input;
    size_t workspace_bytes = 0;
    BufferP workspace;
    BufferP consts;
    std::vector<uint8_t> const_host;
    int fused_ops = 0;
    int launches_estimate = 0;
};

struct IdHash {
    size_t operator()(const std::array<uint8_t, 16>& a) const {
        size_t h = 1469598103934665603ull;
        for (auto b : a) h = (h ^ b) * 1099511628211ull;
        return h;
    }
};

class Backend {
  public:
    explicit Backend(int device);
    ~Backend();

    gptrs_hip_tensor* materialize(const Spec& spec, const void* host, size_t nbytes);
    void to_literal(const gptrs_hip_tensor* t, void* dst, size_t cap);
    void run_program(const char* json, size_t len, uint64_t key, gptrs_hip_tensor* const* inputs,
                     const uint8_t* donate, size_t n_in, gptrs_hip_tensor** outputs, size_t n_out);
    gptrs_hip_tensor* param_get(const std::array<uint8_t, 16>& id);
    void param_set(const std::array<uint8_t, 16>& id, gptrs_hip_tensor* t);
    int64_t sample(const gptrs_hip_tensor* logits, float temperature, bool has_top_k, bool has_u, float u);
    // sample() in two halves for a pipelined decode loop: begin queues the sampling kernels and the copies of the token
    // and of the device error flags into a pinned ring and returns a ticket (-1: request not served here), wait blocks
    // on that ticket's event only.  The token also stays in token_tensor() (si32[1] over the sampling output).
    static constexpr int kTokenRing = 32;
    int64_t sample_begin(const gptrs_hip_tensor* logits, float temperature, bool has_top_k, bool has_u, float u);
    int64_t sample_wait(int64_t ticket);
    gptrs_hip_tensor* token_tensor();
    // the same for a batch: the greedy token of EVERY row of logits [rows <= kMaxTokenRows, vocab]; the tokens stay on
    // the device in rows_tensor(rows) (si32[rows]) and travel to the host through the same ring
    static constexpr int kMaxTokenRows = 64;
    int64_t sample_rows_begin(const gptrs_hip_tensor* logits);
    void sample_rows_wait(int64_t ticket, int32_t* tokens_out, size_t n);
    // greedy token of every row into a caller's si32[rows] tensor; launches only, allocates nothing
    void sample_rows_into(const gptrs_hip_tensor* logits, gptrs_hip_tensor* tokens_out);
    gptrs_hip_tensor* rows_tensor(int64_t rows);
    void synchronize();
    void check_device_errors();

    BufferP new_buffer(size_t bytes);
    // Derived layouts of a weight tensor, built on first use and kept while the source buffer lives
    // (the backend-side memo of derived weight formats).  kind 0: column-tiled copy for the decode
    // GEMV (kernels_gemv_tiled.hip); kind 1: k-grouped copy for the MFMA GEMM (kernels_mfma.hip).
    // kind 2: 4-column / k-pair tiled copy for the persistent decode chain (kernels_chain.hip); with
    // src2 the SwiGLU pair (gate = src, up = src2) interleaved column by column in one copy.
    // Quantised weights: kind 3 / 4: chain copies of int8 / int4 codes (src2: the partner's codes); kind 5:
    // chain copy of int4 group scales (src2: the partner's); kind 6 / 7: k-grouped copy of the int8 / int4
    // codes for the MFMA GEMM, which applies the scales itself; kind 8: 16-column tiled k-grouped copy for batched decode
    // (kernels_skinny.hip); kind 9 / 10: int8 / int4 codes in that tile order; kind 11: chain copy of f32 weights.
    BufferP derived_weights(const BufferP& src, int kind, DType dtype, int64_t k, int64_t n, const BufferP& src2 = nullptr);
    void drop_derived_weights();
    // Row-major weights that a chain copy duplicates: evict_packed_sources frees those among `inputs` that `plan`
    // never reads directly (option "evict_packed_weights", on by default); ensure_resident brings one back, exactly.
    void ensure_resident(const BufferP& b);
    void evict_packed_sources(const Plan& plan, gptrs_hip_tensor* const* inputs, size_t n_in);
    bool opt_evict_weights = true;
    int64_t n_weights_evicted = 0, n_weights_restored = 0;
    // Device copy of a chain's phase table, cached by content (steady-state decode repeats a few tables).
    const k::ChainPhase* chain_table(const std::vector<k::ChainPhase>& phases);
    unsigned* chain_barrier() const { return d_chain_bar_; }
    // kSkinnyTickets zeroed counters behind the chain's (split-K tickets of the batched-decode linear layers)
    unsigned* skinny_tickets() const { return d_chain_bar_ + k::kChainBarrierBytes / sizeof(unsigned); }
    int* chain_abort_flag() const { return d_err_flag_ + 1; }
    bool opt_chain = true;
    // unquantised bf16 prefill linears on the LDS-direct GEMM (option "gemm_lds_direct", GPTRS_HIP_GEMM_DMA); off: the
    // register-staged kernel that also serves f32 and quantised weights
    bool opt_gemm_lds_direct = true;
    // f32 chains run only when a linear phase streams at least this much on average (option "chain_f32_min_kb",
    // GPTRS_HIP_CHAIN_F32_MIN_KB): below it a phase's fixed cost is what a stand-alone kernel costs
    int64_t chain_f32_min_bytes = 4ll << 20;
    int chain_stall_phase = -1;   // tests of the give-up path: the next chain launch expects an arrival too many at this phase
    bool chain_stall_fired = false;   // such a launch has been queued and its time-out not yet reported
    int64_t n_chain_launches = 0, n_chain_phases = 0;
    int64_t n_tiled_built = 0;
    void release_block(void* p, size_t cap) { pool_.release(p, cap); }
    void note_dead_source() { dead_sources_.fetch_add(1, std::memory_order_relaxed); }

    std::mutex mu;
    hipStream_t stream = nullptr;
    int device = 0;
    bool opt_fusion = true;
    // replay steady-state programs (same plan, same buffer addresses) as captured HIP graphs
    bool opt_graphs = true;
    bool capturing = false;
    int64_t n_graph_launches = 0, n_graphs_built = 0, n_graphs_refused = 0;
    // opt-in timing of the linear-layer launches with HIP events on the execution stream
    bool opt_profile = false;
    std::vector<std::pair<hipEvent_t, hipEvent_t>> prof_events;
    int64_t prof_linear_calls = 0, prof_linear_bytes = 0;
    double prof_linear_ns = 0.0;
    void profile_reset();
    void profile_collect();  // synchronises, folds pending event pairs into prof_linear_ns
    // counters
    int64_t n_launches = 0, n_compiled = 0, n_cache_hits = 0, n_fused = 0, n_inplace = 0, last_launches = 0;
    int64_t bytes_allocated() const { return (int64_t)pool_.bytes_allocated; }

  private:
    std::shared_ptr<Plan> get_plan(const char* json, size_t len, uint64_t key, gptrs_hip_tensor* const* inputs, const uint8_t* donate, size_t n_in);
    void execute(Plan& plan, gptrs_hip_tensor* const* inputs, const uint8_t* donate, gptrs_hip_tensor** outputs);
    void tag_broadcast_result(const Plan& plan, size_t r, gptrs_hip_tensor* const* user_inputs, gptrs_hip_tensor* t);
  public:
    void realize(const gptrs_hip_tensor* t);   // gives a lazily broadcast handle its buffer
  private:
    bool run_graphed(Plan& plan, ExecCtx& cx, const std::vector<BufferP>& out_bufs);

    DevicePool pool_;
    std::unordered_map<std::array<uint8_t, 16>, gptrs_hip_tensor*, IdHash> params_;
    std::list<std::pair<uint64_t, std::shared_ptr<Plan>>> plan_lru_;
    std::unordered_map<uint64_t, std::list<std::pair<uint64_t, std::shared_ptr<Plan>>>::iterator> plan_index_;
    // device-side helpers
    int* d_err_flag_ = nullptr;
    int* d_counters_ = nullptr;
    float* d_argmax_val_ = nullptr;
    int32_t* d_argmax_idx_ = nullptr;
    int64_t* d_token_ = nullptr;       // = token_buf_->ptr: the sampled token as int64, little endian
    BufferP token_buf_;
    int64_t* h_token_ring_ = nullptr;  // pinned: kTokenRing x kRingSlot int64: {token, error flags, kMaxTokenRows si32 tokens}
    static constexpr int kRingSlot = 2 + kMaxTokenRows / 2;
    BufferP rows_buf_;                 // si32[kMaxTokenRows]: the tokens of the last sample_rows_begin
    int ring_rows_[kTokenRing] = {};   // rows behind each ticket (0: a single-token ticket)
    hipEvent_t token_events_[kTokenRing] = {};
    int64_t next_ticket_ = 0;
    bool queue_sampling(const gptrs_hip_tensor* logits, float temperature, bool has_top_k, bool has_u, float u);
    void* h_pinned_ = nullptr;  // 64 bytes of pinned host memory for readbacks
    struct Derived { std::weak_ptr<Buffer> src, src2; BufferP tiled; int64_t k = 0, n = 0; };
    std::map<std::array<uint64_t, 3>, Derived> tiled_cache_;
    void forget_chain_copy(const std::array<uint64_t, 3>& key, const Derived& d);
    size_t evicted_since_trim_ = 0;
    std::atomic<int> dead_sources_{0};  // weights with derived layouts that were freed since the last sweep
    unsigned* d_chain_bar_ = nullptr;
    struct ChainTable { std::vector<k::ChainPhase> host; BufferP dev; uint64_t last_use = 0; int refs = 0; };   // refs: recorded graphs that hold its address
    std::vector<const void*> capture_tables_;   // tables looked up while a graph is being recorded
    void release_graph_tables(const PlanGraph& g);
  public:
    int64_t chain_table_count() const { return (int64_t)chain_tables_.size(); }
  private:
    std::vector<ChainTable> chain_tables_;
    uint64_t chain_clock_ = 0;
    uint64_t next_buffer_id_ = 1;
};

void release_handle_locked(gptrs_hip_tensor* t);   // api.cpp

// fuse.cpp: canonicalise + pattern-fuse the entry function in place.  Returns the number of fused ops.
int fuse_function(Function& fn);
// fuse.cpp: inputs that are known broadcasts of a vector.  `src[i]` is the vector's spec for input i (nullptr: an ordinary
// input).  expand: appends one vector parameter per tagged input and makes the body read BroadcastTo(vector) instead of
// the input; returns the positions of the tagged inputs, in the order of the appended parameters.  collapse (after the
// fusion pass): whatever still reads a BroadcastTo that expand inserted reads the input itself again.
struct BroadcastInput { int input = -1; int param_value = -1, bcast_value = -1; };
std::vector<BroadcastInput> expand_broadcast_inputs(Function& fn, const std::vector<const Spec*>& src);
void collapse_broadcast_inputs(Function& fn, const std::vector<BroadcastInput>& expanded);
// fuse.cpp: CustomCall norm targets (norm_call_target) become the FLayerNorm / FRmsNorm instructions the pattern pass
// would have formed from the functional's own sequence; their operands are validated here.  Runs on every program,
// fusion on or off: the targets are part of what the backend executes.
void lower_norm_calls(Function& fn);
// fuse.cpp: the input position whose contents, broadcast along leading axes, are result `r` of the function as written
// (a chain of BroadcastTo / Reshape instructions that keep the last axis), or -1.
int result_broadcast_source(const Function& fn, size_t r);
// plan.cpp: validate every instruction, assign storage and build launch descriptors.
void build_plan(Plan& plan, const std::vector<bool>& donated);
// plan.cpp: run one step with resolved pointers.
struct ExecCtx {
    Backend* be;
    hipStream_t stream;
    std::vector<void*> ptr;  // per value id
    char* ws;
    char* consts;
    int* err_flag;
    int* counters;
    int64_t launches = 0;
    bool profile = false;
    bool chain = false;               // run decode linears as persistent chain launches
    std::vector<BufferP> input_bufs;  // per input position
};
void run_step(const Plan& plan, const Step& st, ExecCtx& cx);

}  // namespace gptrs
