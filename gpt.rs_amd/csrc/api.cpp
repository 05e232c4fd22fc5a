// Backend implementation and the extern "C" surface declared in include/gptrs_hip.h.
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "../../include/gptrs_hip.h"
#include "runtime.hpp"

namespace gptrs {

// ------------------------------------------------------------------------------ device pool
size_t DevicePool::bucket(size_t n) {
    if (n <= 4096) return (n + 255) / 256 * 256;
    size_t p = 4096;
    while (p * 2 <= n) p *= 2;  // p <= n < 2p
    const size_t step = p / 8;
    return (n + step - 1) / step * step;
}
void* DevicePool::alloc(size_t bytes, size_t* cap_out) {
    const size_t cap = bucket(bytes ? bytes : 1);
    *cap_out = cap;
    auto it = free_.find(cap);
    if (it != free_.end() && !it->second.empty()) {
        void* p = it->second.back();
        it->second.pop_back();
        return p;
    }
    void* p = nullptr;
    hipError_t e = hipMalloc(&p, cap);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        trim();
        e = hipMalloc(&p, cap);
        if (e != hipSuccess) fail_exec(std::string("device allocation of ") + std::to_string(cap) + " bytes failed: " + hipGetErrorString(e));
    }
    bytes_allocated += cap;
    return p;
}
void DevicePool::release(void* p, size_t cap) { free_[cap].push_back(p); }
void DevicePool::trim() {
    for (auto& kv : free_) {
        for (void* p : kv.second) { (void)hipFree(p); bytes_allocated -= kv.first; }
        kv.second.clear();
    }
}

Buffer::~Buffer() {
    if (!owner) return;
    if (has_derived) owner->note_dead_source();
    if (ptr) owner->release_block(ptr, cap);
}

// ------------------------------------------------------------------------------ backend
// Drops one reference; the last one frees the handle and lets go of the handles it holds.  The caller holds the owning
// backend's mutex (returning a block to the pool touches backend state).
void release_handle_locked(gptrs_hip_tensor* t) {
    while (t && t->refs.fetch_sub(1) == 1) {
        gptrs_hip_tensor* src = t->bcast_src;
        gptrs_hip_tensor* lazy = t->lazy_input;
        delete t;
        if (lazy) release_handle_locked(lazy);
        t = src;
    }
}

Backend::Backend(int dev) : device(dev) {
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count <= 0)
        fail_exec("no HIP device is visible: the hip backend has no CPU fallback");
    if (dev < 0 || dev >= count) fail_exec("device index out of range");
    GPTRS_HIP_CHECK(hipSetDevice(dev));
    // Graph replay is off when GPTRS_HIP_GRAPHS=0, and under any tool that sits between the runtime and the queues
    // (rocprofv3 and its relatives): a replayed graph under rocprofiler-sdk's kernel tracing was answered with "AQL
    // packet is malformed" and a stalled queue, while the same steps launched one by one trace fine.  The cause is not
    // established (every recorded node passes check_graph_nodes below), so replay stays off whenever a tool may be loaded.
    {
        const char* g = getenv("GPTRS_HIP_GRAPHS");
        bool tool = false;
        for (const char* name : {"ROCP_TOOL_LIBRARIES", "HSA_TOOLS_LIB", "ROCPROFILER_LIBRARY", "ROCTRACER_DOMAIN", "ROCPROFILER_REGISTER_FORCE_LOAD"}) {
            const char* v = getenv(name);
            if (v && v[0]) tool = true;
        }
        const char* pre = getenv("LD_PRELOAD");
        if (pre && (strstr(pre, "rocprof") || strstr(pre, "roctracer") || strstr(pre, "rocprofiler"))) tool = true;
        if ((g && g[0] == '0') || tool) opt_graphs = false;
    }
    GPTRS_HIP_CHECK(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking));
    GPTRS_HIP_CHECK(hipMalloc((void**)&d_err_flag_, 256));
    GPTRS_HIP_CHECK(hipMalloc((void**)&d_counters_, k::kLinearCounters * sizeof(int)));
    GPTRS_HIP_CHECK(k::argmax_noalloc_init(device));   // address of the no-allocation sampling scratch on this GPU
    GPTRS_HIP_CHECK(hipMalloc((void**)&d_argmax_val_, 1024 * sizeof(float)));
    GPTRS_HIP_CHECK(hipMalloc((void**)&d_argmax_idx_, 1024 * sizeof(int32_t)));
    token_buf_ = new_buffer(256);
    d_token_ = (int64_t*)token_buf_->ptr;
    rows_buf_ = new_buffer(kMaxTokenRows * sizeof(int32_t));
    GPTRS_HIP_CHECK(hipHostMalloc((void**)&h_token_ring_, kTokenRing * kRingSlot * sizeof(int64_t), hipHostMallocDefault));
    GPTRS_HIP_CHECK(hipHostMalloc(&h_pinned_, 256, hipHostMallocDefault));
    GPTRS_HIP_CHECK(hipMalloc((void**)&d_chain_bar_, k::kChainBarrierBytes + k::kSkinnyTickets * sizeof(unsigned)));
    k::fill_zero(stream, d_chain_bar_, k::kChainBarrierBytes + k::kSkinnyTickets * sizeof(unsigned));
    {
        const char* c = getenv("GPTRS_HIP_CHAIN");
        if (c && c[0] == '0') opt_chain = false;
        const char* d = getenv("GPTRS_HIP_GEMM_DMA");
        if (d && d[0] == '0') opt_gemm_lds_direct = false;
        if (const char* m = getenv("GPTRS_HIP_CHAIN_F32_MIN_KB")) chain_f32_min_bytes = std::max<int64_t>(0, atoll(m)) << 10;
    }
    k::fill_zero(stream, d_err_flag_, 256);
    k::fill_zero(stream, d_counters_, k::kLinearCounters * sizeof(int));
    GPTRS_HIP_CHECK(hipStreamSynchronize(stream));
}

Backend::~Backend() {
    (void)hipSetDevice(device);
    if (stream) (void)hipStreamSynchronize(stream);
    try { profile_collect(); } catch (...) {}
    for (auto& kv : params_) release_handle_locked(kv.second);
    params_.clear();
    plan_index_.clear();
    plan_lru_.clear();
    tiled_cache_.clear();
    chain_tables_.clear();
    pool_.trim();
    (void)hipFree(d_chain_bar_);
    (void)hipFree(d_err_flag_);
    (void)hipFree(d_counters_);
    (void)hipFree(d_argmax_val_);
    (void)hipFree(d_argmax_idx_);
    token_buf_.reset();
    rows_buf_.reset();
    for (hipEvent_t e : token_events_)
        if (e) (void)hipEventDestroy(e);
    if (h_token_ring_) (void)hipHostFree(h_token_ring_);
    if (h_pinned_) (void)hipHostFree(h_pinned_);
    if (stream) (void)hipStreamDestroy(stream);
}

void Backend::profile_collect() {
    if (prof_events.empty()) return;
    GPTRS_HIP_CHECK(hipStreamSynchronize(stream));
    for (auto& pr : prof_events) {
        float ms = 0.f;
        if (hipEventElapsedTime(&ms, pr.first, pr.second) == hipSuccess) prof_linear_ns += (double)ms * 1e6;
        (void)hipEventDestroy(pr.first);
        (void)hipEventDestroy(pr.second);
    }
    prof_events.clear();
}
void Backend::profile_reset() {
    profile_collect();
    prof_linear_ns = 0.0;
    prof_linear_calls = 0;
    prof_linear_bytes = 0;
}

BufferP Backend::new_buffer(size_t bytes) {
    auto b = std::make_shared<Buffer>();
    b->ptr = pool_.alloc(bytes, &b->cap);
    b->owner = this;
    b->id = next_buffer_id_++;
    return b;
}

BufferP Backend::derived_weights(const BufferP& src, int kind, DType dtype, int64_t k, int64_t n, const BufferP& src2) {
    const std::array<uint64_t, 3> ckey{src->id, src2 ? src2->id : 0, (uint64_t)kind};
    auto it = tiled_cache_.find(ckey);
    if (it != tiled_cache_.end()) {
        if (it->second.src.lock() == src && it->second.src2.lock() == src2) return it->second.tiled;
        forget_chain_copy(it->first, it->second);
        tiled_cache_.erase(it);
    }
    if (capturing) fail_exec("derived weight copy missing while recording a graph");
    // A weight that was freed (a streamed parameter between two forwards) takes its layouts with it, before the next one
    // is built: the memory a caller saves by streaming is not spent on copies of weights that are gone.
    if (dead_sources_.exchange(0, std::memory_order_relaxed) > 0) {
        for (auto e = tiled_cache_.begin(); e != tiled_cache_.end();) {
            if (e->second.src.expired() || (e->first[1] && e->second.src2.expired())) {
                forget_chain_copy(e->first, e->second);   // the surviving half of a pair gets its row-major form back first
                e = tiled_cache_.erase(e);
            } else {
                ++e;
            }
        }
    }
    // every layout is built from the row-major form
    ensure_resident(src);
    ensure_resident(src2);
    BufferP t;
    if (kind == 0) {
        t = new_buffer(k::tiled_weight_bytes((int)dtype, k, n));
        k::tile_weights(stream, (int)dtype, src->ptr, t->ptr, k, n);
    } else if (kind == 1) {
        t = new_buffer(k::mfma_weight_bytes((int)dtype, k, n));
        k::mfma_pack_weights(stream, (int)dtype, src->ptr, t->ptr, k, n);
    } else if (kind == 2 || kind == 3 || kind == 4 || kind == 11) {   // decode chain: bf16 / int8 codes / int4 codes (src2: SwiGLU partner) / f32
        const int wfmt = kind == 11 ? k::kChainW32 : kind - 2;
        t = new_buffer(k::chain_weight_bytes(k, n, src2 != nullptr, wfmt));
        k::chain_pack_weights(stream, src->ptr, src2 ? src2->ptr : nullptr, t->ptr, k, n, wfmt);
    } else if (kind == 5) {                             // decode chain: int4 group scales (src2: the partner's)
        t = new_buffer(k::chain_scale_bytes(k, n, src2 != nullptr));
        k::chain_pack_scales_w4(stream, (int)dtype, src->ptr, src2 ? src2->ptr : nullptr, t->ptr, k, n);
    } else if (kind == 8) {                             // batched decode: 16-column tiles, k-grouped (kernels_skinny.hip)
        t = new_buffer(k::skinny_weight_bytes((int)dtype, k, n));
        k::skinny_pack_weights(stream, (int)dtype, src->ptr, t->ptr, k, n);
    } else if (kind == 9 || kind == 10) {               // batched decode: int8 / int4 codes in the 16-column tiled word order
        t = new_buffer(k::skinny_codes_bytes(k, n, kind - 8));
        k::skinny_pack_codes(stream, src->ptr, t->ptr, k, n, kind - 8);
    } else {                                            // 6 / 7: prefill GEMM: int8 / int4 codes, k-grouped (kernels_mfma.hip)
        t = new_buffer(k::mfma_codes_bytes(k, n, kind - 5));
        k::mfma_pack_codes(stream, src->ptr, t->ptr, k, n, kind - 5);
    }
    Derived d;
    d.src = src;
    src->has_derived = true;
    if (src2) { d.src2 = src2; src2->has_derived = true; }
    d.tiled = t;
    d.k = k;
    d.n = n;
    if (kind == 2) {   // the bf16 chain copy is a permutation of the matrix: enough to rebuild it from
        src->chain_key = ckey;
        if (src2) src2->chain_key = ckey;
    }
    tiled_cache_[ckey] = std::move(d);
    ++n_tiled_built;
    return t;
}

// Called before a chain copy leaves the cache: sources that were evicted in its favour are rebuilt from it first.
void Backend::forget_chain_copy(const std::array<uint64_t, 3>& key, const Derived& d) {
    if (key[2] != 2) return;
    for (BufferP b : {d.src.lock(), d.src2.lock()}) {
        if (!b || b->chain_key != key) continue;
        ensure_resident(b);
        b->chain_key = {{0, 0, 0}};
    }
}

void Backend::ensure_resident(const BufferP& b) {
    if (!b || !b->evicted) return;
    if (capturing) fail_exec("a weight that was evicted in favour of its decode-chain copy is needed while recording a graph");
    auto it = tiled_cache_.find(b->chain_key);
    if (it == tiled_cache_.end() || it->first[2] != 2) fail_exec("an evicted weight has no packed copy left to rebuild it from");
    const BufferP s1 = it->second.src.lock(), s2 = it->second.src2.lock();
    const bool dual = it->first[1] != 0;
    if (s1 != b && !(dual && s2 == b)) fail_exec("an evicted weight is not a source of the packed copy it names");
    size_t cap = 0;
    void* p = pool_.alloc(b->cap, &cap);
    k::chain_unpack_weights(stream, it->second.tiled->ptr, s1 == b ? p : nullptr, dual && s2 == b ? p : nullptr, it->second.k, it->second.n, dual);
    b->ptr = p;
    b->cap = cap;
    b->evicted = false;
    ++n_weights_restored;
}

// After a program ran: inputs that this plan only ever uses through derived layouts, and whose values the bf16 chain
// copy holds as well, give their row-major storage back.  The copy kernels that read them are queued on the one
// stream, ahead of whatever is allocated from the freed blocks later.
void Backend::evict_packed_sources(const Plan& plan, gptrs_hip_tensor* const* inputs, size_t n_in) {
    if (!opt_evict_weights || capturing) return;
    int n = 0;
    for (size_t i = 0; i < n_in && i < plan.input_weight_only.size(); ++i) {
        if (!plan.input_weight_only[i] || !inputs[i]) continue;
        const BufferP& b = inputs[i]->buf;
        if (!b || b->evicted || !b->ptr || b->chain_key[2] != 2) continue;
        // the same tensor passed a second time in a position that reads it: it would be rebuilt on every call
        bool read_elsewhere = false;
        for (size_t j = 0; j < n_in && !read_elsewhere; ++j)
            read_elsewhere = j != i && inputs[j] && inputs[j]->buf == b && !(j < plan.input_weight_only.size() && plan.input_weight_only[j]);
        if (read_elsewhere) continue;
        auto it = tiled_cache_.find(b->chain_key);
        if (it == tiled_cache_.end()) { b->chain_key = {{0, 0, 0}}; continue; }
        if (it->second.src.lock() != b && it->second.src2.lock() != b) continue;
        if (it->first[0] != b->id && it->first[1] != b->id) { b->chain_key = {{0, 0, 0}}; continue; }   // updated in place since: the copy is stale
        pool_.release(b->ptr, b->cap);
        evicted_since_trim_ += b->cap;
        b->ptr = nullptr;
        b->evicted = true;
        ++n;
    }
    n_weights_evicted += n;
    // Back to the driver once it adds up (the point is the process's footprint, not the pool's free list); small
    // amounts stay in the pool, where the next allocation of that size takes them.
    if (n && evicted_since_trim_ >= (size_t)256 << 20) {
        evicted_since_trim_ = 0;
        GPTRS_HIP_CHECK(hipStreamSynchronize(stream));
        pool_.trim();
    }
}

// Frees every derived weight layout (and with them the recorded graphs, which hold their addresses) and returns the
// cached blocks to the driver.  Layouts are built at first use, per kernel family; a caller that is done with one
// family (the prefill copies once a server only decodes) gets their memory back here, the layouts still in use are
// rebuilt by the next call that needs them.
void Backend::drop_derived_weights() {
    GPTRS_HIP_CHECK(hipStreamSynchronize(stream));
    for (auto& kv : plan_lru_) {
        Plan& p = *kv.second;
        for (auto& g : p.graphs) {
            if (g.exec) (void)hipGraphExecDestroy(g.exec);
            if (g.graph) (void)hipGraphDestroy(g.graph);
            release_graph_tables(g);
        }
        p.graphs.clear();
        p.seen_keys.clear();
        p.graph_builds = p.graph_hits = 0;
    }
    for (auto& kv : tiled_cache_) forget_chain_copy(kv.first, kv.second);
    GPTRS_HIP_CHECK(hipStreamSynchronize(stream));
    tiled_cache_.clear();
    pool_.trim();
}

void Backend::release_graph_tables(const PlanGraph& g) {
    for (const void* p : g.tables)
        for (auto& t : chain_tables_)
            if (t.dev->ptr == p) { if (t.refs > 0) --t.refs; break; }
}

const k::ChainPhase* Backend::chain_table(const std::vector<k::ChainPhase>& phases) {
    const size_t bytes = phases.size() * sizeof(k::ChainPhase);
    for (auto& t : chain_tables_)
        if (t.host.size() == phases.size() && !memcmp(t.host.data(), phases.data(), bytes)) {
            t.last_use = ++chain_clock_;
            if (capturing) capture_tables_.push_back(t.dev->ptr);
            return (const k::ChainPhase*)t.dev->ptr;
        }
    if (capturing) fail_exec("chain table missing while recording a graph");
    // A recorded graph keeps the address of its table, so such a table lives as long as the graph.  The others (a
    // launch whose buffer addresses never come back: streamed weights, growing caches) go, least recently used first,
    // once there are 64 of them; the stream orders the reuse of their memory behind the launch that read them.
    size_t loose = 0;
    for (auto& t : chain_tables_) loose += t.refs > 0 ? 0 : 1;
    if (loose >= 64) {
        size_t victim = chain_tables_.size();
        for (size_t i = 0; i < chain_tables_.size(); ++i)
            if (chain_tables_[i].refs == 0 && (victim == chain_tables_.size() || chain_tables_[i].last_use < chain_tables_[victim].last_use)) victim = i;
        chain_tables_.erase(chain_tables_.begin() + (std::ptrdiff_t)victim);
    }
    if (chain_tables_.size() >= 4096) return nullptr;   // (all held by graphs: the caller runs the linears one by one instead)
    ChainTable t;
    t.host = phases;
    t.dev = new_buffer(bytes);
    t.last_use = ++chain_clock_;
    // pageable source: wait, so the vector may go away (tables are built once per address set)
    GPTRS_HIP_CHECK(hipMemcpyAsync(t.dev->ptr, phases.data(), bytes, hipMemcpyHostToDevice, stream));
    GPTRS_HIP_CHECK(hipStreamSynchronize(stream));
    chain_tables_.push_back(std::move(t));
    return (const k::ChainPhase*)chain_tables_.back().dev->ptr;
}

gptrs_hip_tensor* Backend::materialize(const Spec& spec, const void* host, size_t nbytes) {
    GPTRS_HIP_CHECK(hipSetDevice(device));
    const size_t want = spec.bytes();
    if (host && nbytes != want) fail_exec("literal byte length mismatch");
    auto* t = new gptrs_hip_tensor();
    t->spec = spec;
    try {
        t->buf = new_buffer(want);
        if (!want) return t;
        if (!host) {
            k::fill_zero(stream, t->buf->ptr, want);
        } else if (want <= sizeof(k::SmallPayload)) {
            k::SmallPayload p;
            memset(&p, 0, sizeof(p));
            memcpy(p.w, host, want);
            k::store_small(stream, t->buf->ptr, p, (int)want);
        } else {
            // pageable source: the copy is staged by the runtime; wait so the caller may reuse `host`
            GPTRS_HIP_CHECK(hipMemcpyAsync(t->buf->ptr, host, want, hipMemcpyHostToDevice, stream));
            GPTRS_HIP_CHECK(hipStreamSynchronize(stream));
        }
    } catch (...) {
        delete t;
        throw;
    }
    return t;
}

void Backend::check_device_errors() {
    // called after a stream synchronisation
    int* flag = (int*)h_pinned_ + 32;
    GPTRS_HIP_CHECK(hipMemcpyAsync(flag, d_err_flag_, 2 * sizeof(int), hipMemcpyDeviceToHost, stream));
    GPTRS_HIP_CHECK(hipStreamSynchronize(stream));
    if (flag[1]) {
        // a grid barrier of the persistent decode chain gave up: its counters are mid-phase
        k::fill_zero(stream, d_err_flag_, 256);
        k::fill_zero(stream, d_chain_bar_, k::kChainBarrierBytes);
        GPTRS_HIP_CHECK(hipStreamSynchronize(stream));
        if (chain_stall_fired) {   // the stall was asked for (set_option "chain_stall_phase"): one launch, then back to normal
            chain_stall_fired = false;
            fail_exec("decode chain: grid barrier timed out (a stall was requested for this launch); the outputs of the program are invalid");
        }
        opt_chain = false;              // whatever kept the workgroups from meeting would do so again: one kernel per layer from here on
        fail_exec("decode chain: grid barrier timed out (workgroups of one launch were not all resident); the outputs of the program are "
                  "invalid, and this backend runs decode steps one kernel per layer from now on");
    }
    if (flag[0]) {
        k::fill_zero(stream, d_err_flag_, 256);
        fail_exec("take index out of bounds");  // cpu.rs:1632-1634
    }
}

void Backend::to_literal(const gptrs_hip_tensor* t, void* dst, size_t cap) {
    realize(t);
    GPTRS_HIP_CHECK(hipSetDevice(device));
    if (t->consumed) fail_exec("tensor handle was donated to run_program and can no longer be read");
    const size_t n = t->spec.bytes();
    if (cap < n) fail_exec("to_literal destination too small");
    ensure_resident(t->buf);
    if (n) GPTRS_HIP_CHECK(hipMemcpyAsync(dst, t->data(), n, hipMemcpyDeviceToHost, stream));
    GPTRS_HIP_CHECK(hipStreamSynchronize(stream));
    check_device_errors();
}

void Backend::synchronize() {
    GPTRS_HIP_CHECK(hipSetDevice(device));
    GPTRS_HIP_CHECK(hipStreamSynchronize(stream));
    check_device_errors();
}

gptrs_hip_tensor* Backend::param_get(const std::array<uint8_t, 16>& id) {
    auto it = params_.find(id);
    if (it == params_.end()) return nullptr;
    it->second->refs.fetch_add(1);
    return it->second;
}
void Backend::param_set(const std::array<uint8_t, 16>& id, gptrs_hip_tensor* t) {
    t->refs.fetch_add(1);
    auto it = params_.find(id);
    if (it != params_.end()) {
        release_handle_locked(it->second);
        it->second = t;
    } else {
        params_[id] = t;
    }
}

bool Backend::queue_sampling(const gptrs_hip_tensor* logits, float temperature, bool has_top_k, bool has_u, float u) {
    GPTRS_HIP_CHECK(hipSetDevice(device));
    if (logits->consumed) fail_exec("tensor handle was donated to run_program and can no longer be read");
    realize(logits);
    const Spec& s = logits->spec;
    if (!dtype_is_float(s.dtype) || s.rank() < 1 || s.rank() > 2 || s.count() == 0)
        fail_exec("sample_decode_token expects non-empty f32/bf16 logits of rank 1 or 2");
    const int64_t vocab = s.dims.back(), rows = s.rank() == 2 ? s.dims[0] : 1;
    if (has_top_k) return false;  // Ok(None): host sampler handles top-k
    if (temperature <= 0.0f) {
        k::argmax_last_row(stream, (int)s.dtype, logits->data(), rows, vocab, d_token_, d_argmax_val_, d_argmax_idx_, 1024);
        n_launches += 2;
    } else {
        if (!has_u) return false;
        k::sample_temperature_last_row(stream, (int)s.dtype, logits->data(), rows, vocab, temperature, u, d_token_);
        n_launches += 1;
    }
    return true;
}

int64_t Backend::sample(const gptrs_hip_tensor* logits, float temperature, bool has_top_k, bool has_u, float u) {
    if (!queue_sampling(logits, temperature, has_top_k, has_u, u)) return -1;
    int64_t* host = (int64_t*)h_pinned_;
    GPTRS_HIP_CHECK(hipMemcpyAsync(host, d_token_, sizeof(int64_t), hipMemcpyDeviceToHost, stream));
    GPTRS_HIP_CHECK(hipStreamSynchronize(stream));
    check_device_errors();
    return *host;
}

int64_t Backend::sample_begin(const gptrs_hip_tensor* logits, float temperature, bool has_top_k, bool has_u, float u) {
    if (!queue_sampling(logits, temperature, has_top_k, has_u, u)) return -1;
    const int64_t ticket = next_ticket_++;
    const int slot = (int)(ticket % kTokenRing);
    if (!token_events_[slot]) GPTRS_HIP_CHECK(hipEventCreateWithFlags(&token_events_[slot], hipEventDisableTiming));
    ring_rows_[slot] = 0;
    GPTRS_HIP_CHECK(hipMemcpyAsync(h_token_ring_ + kRingSlot * slot, d_token_, sizeof(int64_t), hipMemcpyDeviceToHost, stream));
    GPTRS_HIP_CHECK(hipMemcpyAsync(h_token_ring_ + kRingSlot * slot + 1, d_err_flag_, 2 * sizeof(int), hipMemcpyDeviceToHost, stream));
    GPTRS_HIP_CHECK(hipEventRecord(token_events_[slot], stream));
    return ticket;
}

int64_t Backend::sample_rows_begin(const gptrs_hip_tensor* logits) {
    GPTRS_HIP_CHECK(hipSetDevice(device));
    if (logits->consumed) fail_exec("tensor handle was donated to run_program and can no longer be read");
    realize(logits);
    const Spec& s = logits->spec;
    if (!dtype_is_float(s.dtype) || s.rank() != 2 || s.count() == 0 || s.dims[0] > kMaxTokenRows)
        fail_exec("sample_decode_rows expects non-empty f32/bf16 logits [rows <= 64, vocab]");
    k::argmax_rows(stream, (int)s.dtype, logits->data(), s.dims[0], s.dims[1], (int32_t*)rows_buf_->ptr, d_argmax_val_, d_argmax_idx_, 1024);
    n_launches += 2;
    const int64_t ticket = next_ticket_++;
    const int slot = (int)(ticket % kTokenRing);
    if (!token_events_[slot]) GPTRS_HIP_CHECK(hipEventCreateWithFlags(&token_events_[slot], hipEventDisableTiming));
    ring_rows_[slot] = (int)s.dims[0];
    GPTRS_HIP_CHECK(hipMemcpyAsync(h_token_ring_ + kRingSlot * slot + 2, rows_buf_->ptr, (size_t)s.dims[0] * sizeof(int32_t),
                                   hipMemcpyDeviceToHost, stream));
    GPTRS_HIP_CHECK(hipMemcpyAsync(h_token_ring_ + kRingSlot * slot + 1, d_err_flag_, 2 * sizeof(int), hipMemcpyDeviceToHost, stream));
    GPTRS_HIP_CHECK(hipEventRecord(token_events_[slot], stream));
    return ticket;
}

// The allocation-free variant of sample_rows_begin: kernels only, partial maxima in the library's fixed device array.
void Backend::sample_rows_into(const gptrs_hip_tensor* logits, gptrs_hip_tensor* tokens_out) {
    GPTRS_HIP_CHECK(hipSetDevice(device));
    if (logits->consumed || tokens_out->consumed) fail_exec("tensor handle was donated to run_program and can no longer be used");
    realize(logits);
    realize(tokens_out);
    const Spec& s = logits->spec;
    const int max_rows = k::argmax_noalloc_max_rows();
    if (!dtype_is_float(s.dtype) || s.rank() != 2 || s.count() == 0)
        fail_exec("sample_decode_rows_into expects non-empty f32/bf16 logits [rows, vocab]");
    if (s.dims[0] > max_rows)
        fail_exec("sample_decode_rows_into: " + std::to_string(s.dims[0]) + " rows exceed the fixed scratch of " + std::to_string(max_rows) + " rows");
    if (s.dims[1] > INT32_MAX) fail_exec("sample_decode_rows_into: vocabulary exceeds the si32 token range");
    const Spec& o = tokens_out->spec;
    if (o.dtype != DType::SI32 || o.count() != s.dims[0] || !tokens_out->data())
        fail_exec("sample_decode_rows_into: tokens_out must be si32[rows]");
    if (tokens_out->buf == logits->buf) fail_exec("sample_decode_rows_into: tokens_out and logits are the same buffer");
    if (!k::argmax_rows_noalloc(stream, device, (int)s.dtype, logits->data(), s.dims[0], s.dims[1], (int32_t*)tokens_out->data()))
        fail_exec("sample_decode_rows_into: the scratch of this device is not initialised");
    {
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) fail_exec(std::string("sample_decode_rows_into: kernel launch failed: ") + hipGetErrorString(e));
    }
    if (tokens_out->buf) tokens_out->buf->id = next_buffer_id_++;   // the contents changed
    n_launches += 2;
}

void Backend::sample_rows_wait(int64_t ticket, int32_t* tokens_out, size_t n) {
    if (ticket < 0 || ticket >= next_ticket_ || ticket + kTokenRing <= next_ticket_)
        fail_exec("sample_decode_rows_wait: unknown or expired ticket");
    GPTRS_HIP_CHECK(hipSetDevice(device));
    const int slot = (int)(ticket % kTokenRing);
    if (ring_rows_[slot] == 0 || (size_t)ring_rows_[slot] != n) fail_exec("sample_decode_rows_wait: the ticket holds a different number of rows");
    GPTRS_HIP_CHECK(hipEventSynchronize(token_events_[slot]));
    if (h_token_ring_[kRingSlot * slot + 1] != 0) {
        GPTRS_HIP_CHECK(hipStreamSynchronize(stream));
        check_device_errors();
    }
    memcpy(tokens_out, h_token_ring_ + kRingSlot * slot + 2, n * sizeof(int32_t));
}

gptrs_hip_tensor* Backend::rows_tensor(int64_t rows) {
    if (rows < 1 || rows > kMaxTokenRows) fail_exec("decode_rows_tensor: 1 to 64 rows");
    auto* t = new gptrs_hip_tensor();
    t->spec.dtype = DType::SI32;
    t->spec.dims = {rows};
    t->buf = rows_buf_;
    return t;
}

int64_t Backend::sample_wait(int64_t ticket) {
    if (ticket < 0 || ticket >= next_ticket_ || ticket + kTokenRing <= next_ticket_)
        fail_exec("sample_decode_token_wait: unknown or expired ticket");
    GPTRS_HIP_CHECK(hipSetDevice(device));
    const int slot = (int)(ticket % kTokenRing);
    if (ring_rows_[slot] != 0) fail_exec("sample_decode_token_wait: the ticket belongs to sample_decode_rows_begin");
    GPTRS_HIP_CHECK(hipEventSynchronize(token_events_[slot]));
    if (h_token_ring_[kRingSlot * slot + 1] != 0) {   // a device-side error flag was up when the token was sampled
        GPTRS_HIP_CHECK(hipStreamSynchronize(stream));
        check_device_errors();
    }
    return h_token_ring_[kRingSlot * slot];
}

gptrs_hip_tensor* Backend::token_tensor() {
    auto* t = new gptrs_hip_tensor();
    t->spec.dtype = DType::SI32;
    t->spec.dims = {1};
    t->buf = token_buf_;
    return t;
}

std::shared_ptr<Plan> Backend::get_plan(const char* json, size_t len, uint64_t key, gptrs_hip_tensor* const* inputs, const uint8_t* donate, size_t n_in) {
    uint64_t k2 = key;
    // inputs this backend produced as broadcasts of a vector are planned as BroadcastTo(vector): part of the compiled form
    std::vector<const Spec*> bsrc(n_in, nullptr);
    bool any_bsrc = false;
    if (opt_fusion)
        for (size_t i = 0; i < n_in; ++i)
            if (inputs && inputs[i] && inputs[i]->bcast_src) { bsrc[i] = &inputs[i]->bcast_src->spec; any_bsrc = true; }
    if (key) {
        // donation pattern and fusion switch are part of the compiled form
        k2 = key * 1099511628211ull + (opt_fusion ? 0x9e3779b97f4a7c15ull : 0);
        for (size_t i = 0; i < n_in; ++i) {
            k2 = (k2 ^ (donate && donate[i] ? 0xA5 : 0x11)) * 1099511628211ull;
            if (bsrc[i]) k2 = (k2 ^ (0xB7 + (uint64_t)bsrc[i]->rank())) * 1099511628211ull;
        }
        if (!k2) k2 = 1;
        auto it = plan_index_.find(k2);
        if (it != plan_index_.end()) {
            plan_lru_.splice(plan_lru_.begin(), plan_lru_, it->second);
            ++n_cache_hits;
            return it->second->second;
        }
    }
    std::vector<bool> don(n_in, false);
    for (size_t i = 0; i < n_in; ++i) don[i] = donate && donate[i];
    auto plan = std::make_shared<Plan>();
    plan->fn = parse_program(json, len);
    if (plan->fn.param_ids.size() != n_in) fail_exec("entry input arity mismatch");
    lower_norm_calls(plan->fn);
    {
        // validate the program as written before any rewrite touches it
        Plan check;
        check.fn = plan->fn;
        build_plan(check, don);
    }
    plan->n_user_inputs = n_in;
    plan->result_bcast_input.assign(plan->fn.result_ids.size(), -1);
    for (size_t r = 0; r < plan->fn.result_ids.size(); ++r) plan->result_bcast_input[r] = result_broadcast_source(plan->fn, r);
    if (opt_fusion) {
        std::vector<BroadcastInput> expanded;
        if (any_bsrc) expanded = expand_broadcast_inputs(plan->fn, bsrc);
        for (const BroadcastInput& b : expanded) plan->ext_inputs.push_back(b.input);
        plan->fused_ops = fuse_function(plan->fn);
        collapse_broadcast_inputs(plan->fn, expanded);
        don.resize(plan->fn.param_ids.size(), false);
    }
    build_plan(*plan, don);
    {
        const Function& f = plan->fn;
        plan->input_read.assign(f.param_ids.size(), false);
        auto mark = [&](int v) {
            for (size_t i = 0; i < f.param_ids.size(); ++i)
                if (f.param_ids[i] == v) plan->input_read[i] = true;
        };
        for (const Instr& in : f.body)
            if (!in.dead)
                for (const Operand& o : in.operands)
                    if (o.value >= 0) mark(o.value);
        for (int r : f.result_ids) mark(r);
        // inputs that only ever serve as the weight of an unquantised linear on a derived layout
        std::vector<int> pos_of(plan->values.size(), -1);
        for (size_t i = 0; i < f.param_ids.size(); ++i)
            if (f.param_ids[i] >= 0 && f.param_ids[i] < (int)pos_of.size()) pos_of[f.param_ids[i]] = (int)i;
        std::vector<int> good(f.param_ids.size(), 0), bad(f.param_ids.size(), 0);
        for (const Instr& in : f.body) {
            if (in.dead) continue;
            const bool lin = in.op == OpKind::FLinear && (in.tiled || in.mfma) && !in.quant;
            for (size_t o = 0; o < in.operands.size(); ++o) {
                const int v = in.operands[o].value;
                if (v < 0 || v >= (int)pos_of.size() || pos_of[v] < 0) continue;
                const bool weight = lin && (o == 1 || (in.act == 2 && o == linear_w2_pos(in)));
                ++(weight ? good : bad)[pos_of[v]];
            }
        }
        for (int r : f.result_ids)
            if (r >= 0 && r < (int)pos_of.size() && pos_of[r] >= 0) ++bad[pos_of[r]];
        plan->input_weight_only.assign(f.param_ids.size(), false);
        for (size_t i = 0; i < f.param_ids.size(); ++i) plan->input_weight_only[i] = good[i] > 0 && bad[i] == 0;
    }
    plan->cacheable = key != 0;
    if (plan->workspace_bytes) plan->workspace = new_buffer(plan->workspace_bytes);
    if (!plan->const_host.empty()) {
        plan->consts = new_buffer(plan->const_host.size());
        GPTRS_HIP_CHECK(hipMemcpyAsync(plan->consts->ptr, plan->const_host.data(), plan->const_host.size(), hipMemcpyHostToDevice, stream));
        GPTRS_HIP_CHECK(hipStreamSynchronize(stream));
    }
    ++n_compiled;
    n_fused += plan->fused_ops;
    if (getenv("GPTRS_HIP_DUMP_PLAN")) {
        fprintf(stderr, "[gptrs_hip] plan key=%llx: %zu steps\n", (unsigned long long)key, plan->steps.size());
        for (const Step& st : plan->steps)
            fprintf(stderr, "  %-22s -> %s%s%s\n", st.in.op_name.c_str(), st.in.out_specs[0].str().c_str(),
                    st.chain_len ? (" [chain of " + std::to_string(st.chain_len) + "]").c_str() : "", st.chain_member ? " [chain member]" : "");
    }
    if (key) {
        plan_lru_.emplace_front(k2, plan);
        plan_index_[k2] = plan_lru_.begin();
        while (plan_lru_.size() > 64) {  // program LRU of 64, as the reference arena keeps (plan.rs:20-29)
            for (auto& g : plan_lru_.back().second->graphs) release_graph_tables(g);
            plan_index_.erase(plan_lru_.back().first);
            plan_lru_.pop_back();
        }
    }
    return plan;
}

Plan::~Plan() {
    for (auto& g : graphs) {
        if (g.exec) (void)hipGraphExecDestroy(g.exec);
        if (g.graph) (void)hipGraphDestroy(g.graph);
    }
}

// Every node of a recorded graph against what a queue accepts: kernel nodes with a function, non-empty grids and blocks
// within the device's limits and dynamic LDS within the opt-in maximum; copies and nothing else besides.  A graph that
// fails is not instantiated (the step runs launch by launch).
static bool check_graph_nodes(hipGraph_t graph, int device) {
    size_t n = 0;
    if (hipGraphGetNodes(graph, nullptr, &n) != hipSuccess) return false;
    if (n == 0) return true;
    std::vector<hipGraphNode_t> nodes(n);
    if (hipGraphGetNodes(graph, nodes.data(), &n) != hipSuccess) return false;
    int max_threads = 1024, max_lds = 64 * 1024, max_grid_x = INT32_MAX;
    (void)hipDeviceGetAttribute(&max_threads, hipDeviceAttributeMaxThreadsPerBlock, device);
    (void)hipDeviceGetAttribute(&max_lds, hipDeviceAttributeSharedMemPerBlockOptin, device);
    (void)hipDeviceGetAttribute(&max_grid_x, hipDeviceAttributeMaxGridDimX, device);
    for (size_t i = 0; i < n; ++i) {
        hipGraphNodeType type;
        if (hipGraphNodeGetType(nodes[i], &type) != hipSuccess) return false;
        if (type == hipGraphNodeTypeKernel) {
            hipKernelNodeParams kp{};
            if (hipGraphKernelNodeGetParams(nodes[i], &kp) != hipSuccess) return false;
            const uint64_t threads = (uint64_t)kp.blockDim.x * kp.blockDim.y * kp.blockDim.z;
            if (!kp.func || threads == 0 || threads > (uint64_t)max_threads) return false;
            if (kp.gridDim.x == 0 || kp.gridDim.y == 0 || kp.gridDim.z == 0 || kp.gridDim.x > (unsigned)max_grid_x) return false;
            if ((uint64_t)kp.gridDim.x * kp.blockDim.x > 0xFFFFFFFFull) return false;   // an AQL packet holds the grid in work-items, 32 bits
            if (kp.sharedMemBytes > (unsigned)max_lds) return false;
        } else if (type != hipGraphNodeTypeMemcpy && type != hipGraphNodeTypeEmpty) {
            return false;   // memset nodes in particular: cleared memory goes through fill kernels
        }
    }
    return true;
}

// Steady-state decode runs the same plan over the same addresses every step (weights and KV caches
// stay put, the pool hands the small per-step buffers back in the same order).  Such a step is
// recorded once by stream capture and replayed with one hipGraphLaunch.  An address set is recorded
// the second time it is seen, after an eager run has built every derived weight copy, so nothing is
// allocated while recording.  Returns false when the caller must run the steps eagerly.
bool Backend::run_graphed(Plan& plan, ExecCtx& cx, const std::vector<BufferP>& out_bufs) {
    constexpr size_t kMaxGraphs = 8, kSeenRing = 32;
    if (!opt_graphs || opt_profile || chain_stall_phase >= 0 || chain_stall_fired || !plan.cacheable || plan.steps.size() < 4) return false;
    if (plan.graph_builds >= 16 && plan.graph_hits < 4 * plan.graph_builds) return false;  // addresses never settle
    std::vector<uint64_t> key;
    key.reserve(cx.input_bufs.size() + out_bufs.size() + 8);
    for (const auto& b : cx.input_bufs) key.push_back(b ? (uint64_t)(uintptr_t)b->ptr : 0);
    for (const auto& b : out_bufs) key.push_back((uint64_t)(uintptr_t)b->ptr);
    key.push_back(opt_chain ? 1 : 0);
    key.push_back((uint64_t)chain_f32_min_bytes);
    key.push_back(opt_gemm_lds_direct ? 1 : 0);
    for (const Step& st : plan.steps) {
        if (st.tiled_w_input >= 0) key.push_back(cx.input_bufs[st.tiled_w_input]->id);
        if (st.tiled_w2_input >= 0) key.push_back(cx.input_bufs[st.tiled_w2_input]->id);
        if (st.tiled_s_input >= 0) key.push_back(cx.input_bufs[st.tiled_s_input]->id);
        if (st.tiled_s2_input >= 0) key.push_back(cx.input_bufs[st.tiled_s2_input]->id);
    }
    for (auto& g : plan.graphs)
        if (g.key == key) {
            GPTRS_HIP_CHECK(hipGraphLaunch(g.exec, stream));
            g.last_use = ++plan.graph_clock;
            ++plan.graph_hits;
            ++n_graph_launches;
            cx.launches = g.launches;
            return true;
        }
    uint64_t h = 1469598103934665603ull;
    for (uint64_t v : key) h = (h ^ v) * 1099511628211ull;
    if (std::find(plan.seen_keys.begin(), plan.seen_keys.end(), h) == plan.seen_keys.end()) {
        if (plan.seen_keys.size() < kSeenRing) plan.seen_keys.push_back(h);
        else plan.seen_keys[plan.runs % kSeenRing] = h;
        return false;
    }
    // record
    PlanGraph pg;
    pg.key = std::move(key);
    GPTRS_HIP_CHECK(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
    capture_tables_.clear();
    capturing = true;
    std::string err;
    try {
        for (const Step& st : plan.steps) run_step(plan, st, cx);
    } catch (const std::exception& e) {
        err = e.what();
    }
    capturing = false;
    hipError_t ec = hipStreamEndCapture(stream, &pg.graph);
    if (err.empty() && ec == hipSuccess && pg.graph && !check_graph_nodes(pg.graph, device)) {
        err = "a recorded node is outside what a queue accepts";
        ++n_graphs_refused;
    }
    if (!err.empty() || ec != hipSuccess || !pg.graph) {
        if (pg.graph) (void)hipGraphDestroy(pg.graph);
        (void)hipGetLastError();
        plan.graph_builds += 4;  // a plan that cannot be recorded stops trying soon
        cx.launches = 0;
        return false;
    }
    ec = hipGraphInstantiate(&pg.exec, pg.graph, nullptr, nullptr, 0);
    if (ec != hipSuccess) {
        (void)hipGraphDestroy(pg.graph);
        (void)hipGetLastError();
        plan.graph_builds += 4;
        cx.launches = 0;
        return false;
    }
    pg.launches = cx.launches;
    pg.tables = capture_tables_;
    for (const void* p : pg.tables)
        for (auto& t : chain_tables_)
            if (t.dev->ptr == p) { ++t.refs; break; }
    pg.last_use = ++plan.graph_clock;
    ++plan.graph_builds;
    ++n_graphs_built;
    if (plan.graphs.size() >= kMaxGraphs) {
        auto lru = std::min_element(plan.graphs.begin(), plan.graphs.end(),
                                    [](const PlanGraph& a, const PlanGraph& b) { return a.last_use < b.last_use; });
        (void)hipGraphExecDestroy(lru->exec);
        (void)hipGraphDestroy(lru->graph);
        release_graph_tables(*lru);
        plan.graphs.erase(lru);
    }
    GPTRS_HIP_CHECK(hipGraphLaunch(pg.exec, stream));
    ++n_graph_launches;
    plan.graphs.push_back(std::move(pg));
    return true;
}

void Backend::realize(const gptrs_hip_tensor* t) {
    if (!t || t->buf || !t->lazy_plan) return;
    std::shared_ptr<Plan> plan = std::move(t->lazy_plan);
    gptrs_hip_tensor* in = t->lazy_input;
    t->lazy_input = nullptr;
    gptrs_hip_tensor* out = nullptr;
    try {
        execute(*plan, &in, nullptr, &out);
    } catch (...) {
        t->lazy_plan = plan;
        t->lazy_input = in;
        throw;
    }
    t->buf = out->buf;
    delete out;
    release_handle_locked(in);   // (the caller holds the backend's mutex)
}

void Backend::execute(Plan& plan, gptrs_hip_tensor* const* user_inputs, const uint8_t* user_donate, gptrs_hip_tensor** outputs) {
    const Function& fn = plan.fn;
    const size_t n_in = fn.param_ids.size();
    // the caller's inputs, then the source vectors of the inputs that were planned as broadcasts
    std::vector<gptrs_hip_tensor*> ext(n_in, nullptr);
    std::vector<uint8_t> ext_don(n_in, 0);
    for (size_t i = 0; i < plan.n_user_inputs; ++i) {
        ext[i] = user_inputs[i];
        ext_don[i] = user_donate && user_donate[i];
    }
    for (size_t j = 0; j < plan.ext_inputs.size(); ++j) {
        gptrs_hip_tensor* t = user_inputs[plan.ext_inputs[j]];
        if (!t || !t->bcast_src) fail_exec("input " + std::to_string(plan.ext_inputs[j]) + " lost its broadcast source between planning and execution");
        ext[plan.n_user_inputs + j] = t->bcast_src;
    }
    gptrs_hip_tensor* const* inputs = ext.data();
    const uint8_t* donate = user_donate ? ext_don.data() : nullptr;
    for (size_t i = 0; i < n_in; ++i) {
        if (!inputs[i]) fail_exec("null input handle");
        if (inputs[i]->consumed) fail_exec("input " + std::to_string(i) + " was donated to an earlier run_program call");
        if (inputs[i]->spec != fn.param_specs[i])
            fail_exec("entry input " + std::to_string(i) + " is " + inputs[i]->spec.str() + " but the program expects " + fn.param_specs[i].str());
        if (plan.input_read[i]) realize(inputs[i]);
        if (!plan.input_weight_only[i]) ensure_resident(inputs[i]->buf);   // some kernel reads the row-major storage
    }
    // a buffer donated for in-place update must not be reachable through another input or handle
    std::vector<bool> inplace_ok(n_in, false);
    for (size_t ob = 0; ob < plan.out_buffer_inplace_input.size(); ++ob) {
        const int ip = plan.out_buffer_inplace_input[ob];
        if (ip < 0) continue;
        bool ok = donate && donate[ip] && inputs[ip]->refs.load() == 1 && inputs[ip]->buf.use_count() == 1;
        for (size_t j = 0; j < n_in && ok; ++j)
            if ((int)j != ip && inputs[j]->buf && inputs[j]->buf == inputs[ip]->buf) ok = false;
        inplace_ok[ip] = ok;
    }
    // output buffers
    std::vector<BufferP> out_bufs(plan.out_buffer_bytes.size());
    for (size_t ob = 0; ob < out_bufs.size(); ++ob) {
        const int ip = plan.out_buffer_inplace_input[ob];
        if (ip >= 0 && inplace_ok[ip]) {
            out_bufs[ob] = inputs[ip]->buf;
            ++n_inplace;
        } else {
            out_bufs[ob] = new_buffer(plan.out_buffer_bytes[ob]);
        }
    }
    ExecCtx cx;
    cx.be = this;
    cx.stream = stream;
    cx.ws = plan.workspace ? (char*)plan.workspace->ptr : nullptr;
    cx.consts = plan.consts ? (char*)plan.consts->ptr : nullptr;
    cx.err_flag = d_err_flag_;
    cx.counters = d_counters_;
    cx.profile = opt_profile;
    cx.chain = opt_chain && k::chain_grid() > 0;
    cx.input_bufs.resize(n_in);
    for (size_t i = 0; i < n_in; ++i) cx.input_bufs[i] = inputs[i]->buf;
    cx.ptr.assign(plan.values.size(), nullptr);
    for (size_t v = 0; v < plan.values.size(); ++v) {
        if (!plan.values[v].defined) continue;
        int r = plan.values[v].root;
        while (plan.values[r].root != r) r = plan.values[r].root;
        const RootStorage& rs = plan.storage[r];
        switch (rs.kind) {
            case Storage::Input: cx.ptr[v] = inputs[rs.index]->data(); break;
            case Storage::Output: cx.ptr[v] = out_bufs[rs.index]->ptr; break;
            case Storage::Const: cx.ptr[v] = cx.consts + rs.offset; break;
            case Storage::Temp: cx.ptr[v] = cx.ws ? cx.ws + rs.offset : nullptr; break;
            case Storage::InPlace: break;
        }
    }
    // From here on kernels that update donated inputs in place may be queued: whatever happens next, those handles no
    // longer hold what the caller gave (an error below leaves them consumed rather than silently changed).
    auto consume_donated = [&]() {
        for (size_t ip = 0; ip < n_in; ++ip)
            if (inplace_ok[ip] && !inputs[ip]->consumed) {
                inputs[ip]->consumed = true;
                inputs[ip]->buf->id = next_buffer_id_++;  // contents changed: derived copies are stale
            }
    };
    try {
        if (!run_graphed(plan, cx, out_bufs))
            for (const Step& st : plan.steps) run_step(plan, st, cx);
        ++plan.runs;
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) fail_exec(std::string("kernel launch failed: ") + hipGetErrorString(e));
    } catch (...) {
        consume_donated();
        throw;
    }
    n_launches += cx.launches;
    last_launches = cx.launches;
    // results
    for (size_t i = 0; i < fn.result_ids.size(); ++i) {
        auto* t = new gptrs_hip_tensor();
        t->spec = fn.result_specs[i];
        if (plan.result_input_alias[i] >= 0) t->buf = inputs[plan.result_input_alias[i]]->buf;
        else t->buf = out_bufs[plan.out_buffer_of_result[i]];
        tag_broadcast_result(plan, i, user_inputs, t);
        outputs[i] = t;
    }
    consume_donated();
    evict_packed_sources(plan, inputs, n_in);
}

// A result that is a pure broadcast of input p along leading axes remembers the vector it came from.
static gptrs_hip_tensor* broadcast_root(gptrs_hip_tensor* in) { return in->bcast_src ? in->bcast_src : in; }
void Backend::tag_broadcast_result(const Plan& plan, size_t r, gptrs_hip_tensor* const* user_inputs, gptrs_hip_tensor* t) {
    const int p = r < plan.result_bcast_input.size() ? plan.result_bcast_input[r] : -1;
    if (p < 0 || !user_inputs[p]) return;
    t->bcast_src = broadcast_root(user_inputs[p]);
    t->bcast_src->refs.fetch_add(1);
}

void Backend::run_program(const char* json, size_t len, uint64_t key, gptrs_hip_tensor* const* inputs,
                          const uint8_t* donate, size_t n_in, gptrs_hip_tensor** outputs, size_t n_out) {
    GPTRS_HIP_CHECK(hipSetDevice(device));
    auto plan = get_plan(json, len, key, inputs, donate, n_in);
    if (plan->fn.result_ids.size() != n_out)
        fail_exec("program produces " + std::to_string(plan->fn.result_ids.size()) + " results but " + std::to_string(n_out) + " were requested");
    // One input, one result, the result a broadcast of the input (the subgraph the reference's parameter-only fold runs
    // for a norm gain or a bias): nothing is computed until something reads the broadcast data itself.
    if (opt_fusion && n_in == 1 && n_out == 1 && plan->result_bcast_input[0] == 0 && inputs[0] && !inputs[0]->consumed &&
        inputs[0]->spec == plan->fn.param_specs[0] && !(donate && donate[0])) {
        auto* t = new gptrs_hip_tensor();
        t->spec = plan->fn.result_specs[0];
        t->backend = this;
        t->lazy_plan = plan;
        t->lazy_input = inputs[0];
        inputs[0]->refs.fetch_add(1);
        tag_broadcast_result(*plan, 0, inputs, t);
        outputs[0] = t;
        last_launches = 0;
        return;
    }
    execute(*plan, inputs, donate, outputs);
}

}  // namespace gptrs

// ================================================================================ C ABI
using gptrs::Backend;
using gptrs::BackendError;

struct gptrs_hip_backend {
    Backend impl;
    explicit gptrs_hip_backend(int dev) : impl(dev) {}
};

static thread_local std::string g_last_error;

template <typename F>
static int guarded(F&& f) {
    try {
        f();
        return GPTRS_HIP_OK;
    } catch (const BackendError& e) {
        g_last_error = e.what();
        return (int)e.kind;
    } catch (const std::exception& e) {
        g_last_error = std::string("backend execution failure: ") + e.what();
        return GPTRS_HIP_ERR_EXECUTION;
    }
}

static gptrs::Spec spec_from_desc(const gptrs_hip_tensor_desc* d) {
    if (!d) gptrs::fail_exec("null tensor descriptor");
    gptrs::Spec s;
    switch (d->dtype) {
        case GPTRS_HIP_F32: s.dtype = gptrs::DType::F32; break;
        case GPTRS_HIP_BF16: s.dtype = gptrs::DType::BF16; break;
        case GPTRS_HIP_SI32: s.dtype = gptrs::DType::SI32; break;
        case GPTRS_HIP_I1: s.dtype = gptrs::DType::I1; break;
        case GPTRS_HIP_SI8: s.dtype = gptrs::DType::SI8; break;
        case GPTRS_HIP_UI8: s.dtype = gptrs::DType::UI8; break;
        default: gptrs::fail_spec("dtype_not_supported (dtype tag " + std::to_string(d->dtype) + ")");
    }
    if (d->rank > 8) gptrs::fail_spec("rank above 8");
    for (uint32_t i = 0; i < d->rank; ++i) {
        if (d->dims[i] < 0) gptrs::fail_spec("negative dimension");
        s.dims.push_back(d->dims[i]);
    }
    return s;
}

extern "C" {

int gptrs_hip_create(int device, gptrs_hip_backend** out) {
    return guarded([&] {
        if (!out) gptrs::fail_exec("null output pointer");
        *out = new gptrs_hip_backend(device);
    });
}

void gptrs_hip_destroy(gptrs_hip_backend* b) { delete b; }

const char* gptrs_hip_backend_name(const gptrs_hip_backend*) { return "hip"; }

int gptrs_hip_materialize(gptrs_hip_backend* b, const gptrs_hip_tensor_desc* desc, const void* host_bytes, size_t nbytes,
                          gptrs_hip_tensor** out) {
    return guarded([&] {
        if (!b || !out) gptrs::fail_exec("null argument");
        const gptrs::Spec s = spec_from_desc(desc);
        std::lock_guard<std::mutex> g(b->impl.mu);
        *out = b->impl.materialize(s, host_bytes, nbytes);
    });
}

int gptrs_hip_to_literal(gptrs_hip_backend* b, const gptrs_hip_tensor* t, void* host_dst, size_t cap) {
    return guarded([&] {
        if (!b || !t || (!host_dst && cap)) gptrs::fail_exec("null argument");
        std::lock_guard<std::mutex> g(b->impl.mu);
        b->impl.to_literal(t, host_dst, cap);
    });
}

void gptrs_hip_tensor_retain(gptrs_hip_tensor* t) {
    if (t) t->refs.fetch_add(1);
}

void gptrs_hip_tensor_release(gptrs_hip_tensor* t) {
    if (!t) return;
    gptrs::Backend* owner = t->buf ? t->buf->owner : t->backend;
    if (owner) {
        std::lock_guard<std::mutex> g(owner->mu);
        gptrs::release_handle_locked(t);
    } else {
        gptrs::release_handle_locked(t);
    }
}

int gptrs_hip_tensor_spec(const gptrs_hip_tensor* t, uint32_t* dtype_out, int64_t* dims_out, size_t dims_cap) {
    if (!t) return -1;
    if (dtype_out) *dtype_out = (uint32_t)t->spec.dtype;
    for (size_t i = 0; i < t->spec.dims.size() && i < dims_cap; ++i) dims_out[i] = t->spec.dims[i];
    return t->spec.rank();
}

int gptrs_hip_run_program_donate(gptrs_hip_backend* b, const char* program_json, size_t json_len, uint64_t program_key,
                                 gptrs_hip_tensor* const* inputs, const uint8_t* donate, size_t n_in,
                                 gptrs_hip_tensor** outputs, size_t n_out) {
    return guarded([&] {
        if (!b || !program_json || (n_in && !inputs) || (n_out && !outputs)) gptrs::fail_exec("null argument");
        std::lock_guard<std::mutex> g(b->impl.mu);
        b->impl.run_program(program_json, json_len, program_key, inputs, donate, n_in, outputs, n_out);
    });
}

int gptrs_hip_run_program(gptrs_hip_backend* b, const char* program_json, size_t json_len, uint64_t program_key,
                          gptrs_hip_tensor* const* inputs, size_t n_in, gptrs_hip_tensor** outputs, size_t n_out) {
    return gptrs_hip_run_program_donate(b, program_json, json_len, program_key, inputs, nullptr, n_in, outputs, n_out);
}

int gptrs_hip_execute_instruction(gptrs_hip_backend* b, const char* instruction_json, size_t json_len,
                                  gptrs_hip_tensor* const* inputs, size_t n_in, gptrs_hip_tensor** output) {
    return guarded([&] {
        if (!b || !instruction_json || !output) gptrs::fail_exec("null argument");
        // Wrap the instruction into a one-instruction program whose parameters are the Value
        // operands in order of appearance.
        gptrs::Json j;
        try {
            j = gptrs::JsonParser(instruction_json, json_len).parse();
        } catch (const gptrs::JsonError& e) {
            gptrs::fail_spec(e.what());
        }
        std::string params, ids;
        size_t nv = 0;
        // inputs are positional, one per Value operand (spec.rs:1317); an id that repeats (x * x) names one parameter
        std::vector<std::pair<int64_t, gptrs_hip_tensor*>> seen;
        std::vector<gptrs_hip_tensor*> uniq;
        try {
            for (auto& od : j.at("operands").as_array())
                if (const gptrs::Json* v = od.find("Value")) {
                    if (nv >= n_in) gptrs::fail_exec("execute_instruction: fewer inputs than Value operands");
                    if (!inputs[nv]) gptrs::fail_exec("null input handle");
                    const int64_t id = v->as_int();
                    bool dup = false;
                    for (auto& pr : seen)
                        if (pr.first == id) {
                            if (pr.second != inputs[nv]) gptrs::fail_exec("execute_instruction: one value id bound to two tensors");
                            dup = true;
                        }
                    ++nv;
                    if (dup) continue;
                    seen.push_back({id, inputs[nv - 1]});
                    uniq.push_back(inputs[nv - 1]);
                    const gptrs::Spec& s = inputs[nv - 1]->spec;
                    std::string dims;
                    for (size_t i = 0; i < s.dims.size(); ++i) dims += (i ? "," : "") + std::string("{\"Static\":") + std::to_string(s.dims[i]) + "}";
                    params += (uniq.size() > 1 ? "," : "") + std::string("{\"Tensor\":{\"dtype\":\"") + gptrs::dtype_name(s.dtype) + "\",\"shape\":{\"dims\":[" + dims + "]}}}";
                    ids += (uniq.size() > 1 ? "," : "") + std::to_string(id);
                }
        } catch (const gptrs::JsonError& e) {
            gptrs::fail_spec(e.what());
        }
        if (nv != n_in) gptrs::fail_exec("execute_instruction: input count does not match Value operands");
        // result type = the instruction's own output
        const char* p = strstr(instruction_json, "\"output\"");
        if (!p) gptrs::fail_spec("json error: missing field `output`");
        const char* colon = strchr(p, ':');
        int depth = 0;
        const char* q = colon + 1;
        const char* start = nullptr;
        const char* end_all = instruction_json + json_len;
        for (; q < end_all; ++q) {
            if (*q == '{') { if (!depth) start = q; ++depth; }
            else if (*q == '}') { --depth; if (!depth) { ++q; break; } }
        }
        if (!start) gptrs::fail_spec("json error: malformed `output`");
        const std::string out_type(start, q);
        const std::string prog = std::string("{\"spec_version\":\"ptir.v0.4\",\"entry\":\"main\",\"functions\":[{\"name\":\"main\",\"parameters\":[") +
                                 params + "],\"parameter_ids\":[" + ids + "],\"results\":[" + out_type + "],\"body\":[" +
                                 std::string(instruction_json, json_len) + "],\"hints\":[],\"result_ids\":[" +
                                 std::to_string(j.at("id").as_int()) + "]}],\"regions\":[]}";
        std::lock_guard<std::mutex> g(b->impl.mu);
        b->impl.run_program(prog.data(), prog.size(), 0, uniq.data(), nullptr, uniq.size(), output, 1);
    });
}

int gptrs_hip_param_get(gptrs_hip_backend* b, const uint8_t id[16], gptrs_hip_tensor** out) {
    return guarded([&] {
        if (!b || !id || !out) gptrs::fail_exec("null argument");
        std::array<uint8_t, 16> key;
        memcpy(key.data(), id, 16);
        std::lock_guard<std::mutex> g(b->impl.mu);
        *out = b->impl.param_get(key);
    });
}

int gptrs_hip_param_set(gptrs_hip_backend* b, const uint8_t id[16], gptrs_hip_tensor* t) {
    return guarded([&] {
        if (!b || !id || !t) gptrs::fail_exec("null argument");
        std::array<uint8_t, 16> key;
        memcpy(key.data(), id, 16);
        std::lock_guard<std::mutex> g(b->impl.mu);
        b->impl.param_set(key, t);
    });
}

int gptrs_hip_supports_decode_sampling(const gptrs_hip_backend*, float temperature, int has_top_k, int has_random_u) {
    if (has_top_k) return 0;
    return temperature <= 0.0f || has_random_u ? 1 : 0;
}

int gptrs_hip_sample_decode_token(gptrs_hip_backend* b, const gptrs_hip_tensor* logits, float temperature, int has_top_k,
                                  int has_random_u, float random_u, int64_t* token_out) {
    return guarded([&] {
        if (!b || !logits || !token_out) gptrs::fail_exec("null argument");
        std::lock_guard<std::mutex> g(b->impl.mu);
        *token_out = b->impl.sample(logits, temperature, has_top_k != 0, has_random_u != 0, random_u);
    });
}

int gptrs_hip_sample_decode_token_begin(gptrs_hip_backend* b, const gptrs_hip_tensor* logits, float temperature, int has_top_k,
                                        int has_random_u, float random_u, int64_t* ticket_out) {
    return guarded([&] {
        if (!b || !logits || !ticket_out) gptrs::fail_exec("null argument");
        std::lock_guard<std::mutex> g(b->impl.mu);
        *ticket_out = b->impl.sample_begin(logits, temperature, has_top_k != 0, has_random_u != 0, random_u);
    });
}

int gptrs_hip_sample_decode_token_wait(gptrs_hip_backend* b, int64_t ticket, int64_t* token_out) {
    return guarded([&] {
        if (!b || !token_out) gptrs::fail_exec("null argument");
        std::lock_guard<std::mutex> g(b->impl.mu);
        *token_out = b->impl.sample_wait(ticket);
    });
}

int gptrs_hip_sample_decode_rows_begin(gptrs_hip_backend* b, const gptrs_hip_tensor* logits, int64_t* ticket_out) {
    return guarded([&] {
        if (!b || !logits || !ticket_out) gptrs::fail_exec("null argument");
        std::lock_guard<std::mutex> g(b->impl.mu);
        *ticket_out = b->impl.sample_rows_begin(logits);
    });
}

int gptrs_hip_sample_decode_rows_into(gptrs_hip_backend* b, const gptrs_hip_tensor* logits, gptrs_hip_tensor* tokens_out) {
    return guarded([&] {
        if (!b || !logits || !tokens_out) gptrs::fail_exec("null argument");
        std::lock_guard<std::mutex> g(b->impl.mu);
        b->impl.sample_rows_into(logits, tokens_out);
    });
}

int gptrs_hip_sample_decode_rows_wait(gptrs_hip_backend* b, int64_t ticket, int32_t* tokens_out, size_t n) {
    return guarded([&] {
        if (!b || !tokens_out) gptrs::fail_exec("null argument");
        std::lock_guard<std::mutex> g(b->impl.mu);
        b->impl.sample_rows_wait(ticket, tokens_out, n);
    });
}

int gptrs_hip_decode_rows_tensor(gptrs_hip_backend* b, int64_t rows, gptrs_hip_tensor** out) {
    return guarded([&] {
        if (!b || !out) gptrs::fail_exec("null argument");
        std::lock_guard<std::mutex> g(b->impl.mu);
        *out = b->impl.rows_tensor(rows);
    });
}

int gptrs_hip_decode_token_tensor(gptrs_hip_backend* b, gptrs_hip_tensor** out) {
    return guarded([&] {
        if (!b || !out) gptrs::fail_exec("null argument");
        std::lock_guard<std::mutex> g(b->impl.mu);
        *out = b->impl.token_tensor();
    });
}

const char* gptrs_hip_last_error(void) { return g_last_error.c_str(); }

int gptrs_hip_fusion_report(const char* program_json, size_t json_len, const int64_t* bcast_len, size_t n_in, char* out, size_t cap,
                            size_t* needed) {
    return guarded([&] {
        if (!program_json || !needed) gptrs::fail_exec("null argument");
        gptrs::Function fn = gptrs::parse_program(program_json, json_len);
        if (fn.param_ids.size() != n_in) gptrs::fail_exec("entry input arity mismatch");
        gptrs::lower_norm_calls(fn);
        std::vector<gptrs::Spec> vec(n_in);
        std::vector<const gptrs::Spec*> src(n_in, nullptr);
        for (size_t i = 0; i < n_in; ++i)
            if (bcast_len && bcast_len[i] > 0) {
                vec[i].dtype = fn.param_specs[i].dtype;
                vec[i].dims = {bcast_len[i]};
                src[i] = &vec[i];
            }
        const std::vector<gptrs::BroadcastInput> expanded = gptrs::expand_broadcast_inputs(fn, src);
        gptrs::fuse_function(fn);
        gptrs::collapse_broadcast_inputs(fn, expanded);
        std::string text;
        for (const gptrs::Instr& in : fn.body) {
            if (in.dead) continue;
            text += in.op_name;
            if (in.op == gptrs::OpKind::FLinear) {
                if (in.norm) text += in.norm_ln ? "+layer_norm" : "+rms_norm";
                if (in.has_bias) text += "+bias";
                if (in.act == 1) text += "+gelu";
                if (in.act == 2) text += "+swiglu";
                if (in.has_residual) text += "+residual";
                text += in.mfma ? " [gemm]" : in.tiled ? " [stream]" : " [generic]";
            }
            if (in.op == gptrs::OpKind::FAttnDecode && in.rot_half > 0) text += "+rope";
            text += '\n';
        }
        *needed = text.size() + 1;
        if (out && cap) {
            const size_t n = std::min(cap - 1, text.size());
            memcpy(out, text.data(), n);
            out[n] = 0;
        }
    });
}

int gptrs_hip_synchronize(gptrs_hip_backend* b) {
    return guarded([&] {
        if (!b) gptrs::fail_exec("null argument");
        std::lock_guard<std::mutex> g(b->impl.mu);
        b->impl.synchronize();
    });
}

int gptrs_hip_set_option(gptrs_hip_backend* b, const char* name, int64_t value) {
    return guarded([&] {
        if (!b || !name) gptrs::fail_exec("null argument");
        std::lock_guard<std::mutex> g(b->impl.mu);
        if (!strcmp(name, "fusion")) b->impl.opt_fusion = value != 0;
        else if (!strcmp(name, "graphs")) b->impl.opt_graphs = value != 0;
        else if (!strcmp(name, "chain")) b->impl.opt_chain = value != 0;
        else if (!strcmp(name, "gemm_lds_direct")) b->impl.opt_gemm_lds_direct = value != 0;
        else if (!strcmp(name, "chain_f32_min_kb")) b->impl.chain_f32_min_bytes = std::max<int64_t>(0, value) << 10;
        else if (!strcmp(name, "chain_stall_phase")) {
            // phase 0 has no barrier in front of it: a stall there would never fire and the option would stay armed
            if (value == 0) gptrs::fail_spec("chain_stall_phase must be >= 1 (or negative to disarm)");
            b->impl.chain_stall_phase = value < 0 ? -1 : (int)std::min<int64_t>(value, 1 << 20);
        }
        else if (!strcmp(name, "profile")) { b->impl.profile_reset(); b->impl.opt_profile = value != 0; }
        else if (!strcmp(name, "drop_derived_weights")) { if (value) b->impl.drop_derived_weights(); }
        else if (!strcmp(name, "evict_packed_weights")) b->impl.opt_evict_weights = value != 0;
        else gptrs::fail_spec(std::string("unknown option `") + name + "`");
    });
}

int64_t gptrs_hip_counter(const gptrs_hip_backend* b, const char* name) {
    if (!b || !name) return -1;
    if (!strncmp(name, "linear_", 7)) {
        Backend& m = const_cast<Backend&>(b->impl);
        std::lock_guard<std::mutex> g(m.mu);
        try { m.profile_collect(); } catch (...) { return -1; }
        if (!strcmp(name, "linear_time_ns")) return (int64_t)m.prof_linear_ns;
        if (!strcmp(name, "linear_calls")) return m.prof_linear_calls;
        if (!strcmp(name, "linear_bytes")) return m.prof_linear_bytes;
        return -1;
    }
    const Backend& i = b->impl;
    if (!strcmp(name, "kernel_launches")) return i.n_launches;
    if (!strcmp(name, "programs_compiled")) return i.n_compiled;
    if (!strcmp(name, "program_cache_hits")) return i.n_cache_hits;
    if (!strcmp(name, "fused_ops")) return i.n_fused;
    if (!strcmp(name, "bytes_allocated")) return i.bytes_allocated();
    if (!strcmp(name, "inplace_updates")) return i.n_inplace;
    if (!strcmp(name, "derived_weights_built")) return i.n_tiled_built;
    if (!strcmp(name, "weights_evicted")) return i.n_weights_evicted;
    if (!strcmp(name, "weights_restored")) return i.n_weights_restored;
    if (!strcmp(name, "last_program_launches")) return i.last_launches;
    if (!strcmp(name, "graph_launches")) return i.n_graph_launches;
    if (!strcmp(name, "graphs_built")) return i.n_graphs_built;
    if (!strcmp(name, "graphs_refused")) return i.n_graphs_refused;
    if (!strcmp(name, "chain_launches")) return i.n_chain_launches;
    if (!strcmp(name, "chain_phases")) return i.n_chain_phases;
    if (!strcmp(name, "chain_tables")) return i.chain_table_count();
    return -1;
}

}  // extern "C"
