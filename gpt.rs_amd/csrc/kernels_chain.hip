// Decode linear layers as ONE persistent launch per run of consecutive linears ("chain").
//
// A decode step of a transformer block is a dependent sequence of GEMVs (out-proj -> gate/up ->
// down -> next block's qkv ...), each streaming tens of MB of weights once.  Launched one by one,
// every GEMV pays a launch gap, a cold start and a tail; here the whole run executes inside one
// kernel of one workgroup per CU, phases separated by a grid-wide barrier:
//
//   * 8 compute waves per workgroup stream the workgroup's weight words from HBM straight into LDS
//     (global_load_lds_dwordx4: no registers), each wave into a ring of its own (3 KiB per j-step: one 16-byte
//     word per lane and tile of the unit), in the order they are consumed: phase by phase, unit by unit (TP
//     tiles of 4 output columns for the whole of K), j-step by j-step.  Weights do not depend on activations,
//     so a wave's requests run four or five j-steps ahead of its reads across unit AND phase boundaries: while the
//     wave stands at the grid barrier, stages the next input or runs an attention phase, HBM keeps delivering
//     the next phase's first words.  Loads of a wave return in order, so "j-step g has landed" is a wait on
//     the count of loads in flight: a ring private to the wave needs no flags and no barrier.  The loop
//     around a j-step is kept to a few dozen instructions (uniform bookkeeping in scalar registers, one vector
//     add and clamp per request): with three waves per SIMD a longer loop body, not HBM, sets the pace.
//   * the compute lanes read their words from the ring (lane t owns word t of each tile stream,
//     Wc[tile][k/2][4 cols][2 k]) and issue v_dot2 (bf16 pairs) against the activation vector staged in LDS.
//   * 1 control wave per workgroup sums the 8 waves' partial sums of a unit out of LDS, applies the
//     epilogue (SwiGLU pair, bias, GELU, residual), stores through to memory, and runs the grid
//     barrier (16 striped arrival counters, one poll instruction).
//   * Activations cross workgroups through agent-scope (sc1) loads and stores only, so no
//     L2 write-back / invalidate is needed between phases; a phase's input vector is staged into
//     LDS by the 9 compute and control waves together right after the barrier (RMSNorm statistics
//     included).
//   * Phase descriptors are read from the table in memory ahead of the wait that precedes their use (scalar
//     loads in the compute waves, one vector load with a lane per dword in the control wave), so a phase opens
//     the moment its barrier is seen.
//
// Decode attention (T = 1 over the KV cache) runs inside the same launch as two more phase kinds,
// executed by all 9 waves of a workgroup together: "partial" (one workgroup per kv head and
// position chunk: append this step's K/V row, online softmax over the chunk for the query heads
// of the group) and "combine" (one workgroup per query head merges the chunk records).
//
// Weight-only quantised linears stream the same 16-byte words with more k per word: int8 codes
// (4 columns x 4 k, stored biased by 128) and int4 codes (4 columns x 8 k, biased by 8, with one bf16
// scale per column and group of 128 k fetched beside the word).  Codes are converted with the
// unsigned-byte converts and accumulated in f32 against the bf16 activations (every product is
// exact); the bias is taken out per word (-128 or -8 times the sum of the word's activations), the
// per-column int8 scale is applied by the control wave.
//
// Every wait is bounded by wall-clock time: a barrier that does not complete raises the abort flag, every
// wave leaves the kernel, and the host reports an execution error.
#include <algorithm>
#include <climits>
#include <cstddef>
#include <cstdlib>
#include <type_traits>

#include "kernels.hpp"
#include "device_utils.hpp"

namespace gptrs {
namespace k {

namespace {

constexpr int NS = 512;          // compute threads
constexpr int NT = NS + 64;      // + control wave: the threads that stage inputs and run attention phases
constexpr int NWS = NS / 64;
constexpr int TP = 3;            // tiles (of 4 columns) per unit
constexpr int NSLOT = 4;         // unit hand-off slots between compute waves and control wave
constexpr int NC = kChainCounters;
constexpr int EPI_MAX = 640;     // bias/residual values staged per workgroup and phase: N <= 160 * grid columns
constexpr int MAXI = 8;          // 8-byte items per thread in the norm staging: K <= 4*MAXI*NT
constexpr int SLOT_BYTES = TP * NS * 16;     // one j-step of a workgroup: a word per compute lane and tile
constexpr int PARK_W4 = 1, PARK_W8 = 2;   // ... in the int4 and int8 kernels, whose step arithmetic and staging hold more registers (measured: one step more spills)
constexpr int PARK = 3;             // j-steps a compute wave can hold in registers while it waits for a phase to open
constexpr int RING_MIN = 4, RING_MAX = 5;    // j-steps a wave's ring holds (its requests run that far ahead of its reads): 5 where the staged activations leave room
constexpr int LDS_BYTES = 160 * 1024;        // per workgroup on gfx950
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }
// The thread index behind an opaque barrier: values derived from it are recomputed by the phase that uses them instead of
// being computed once per launch and held in registers (or spilled) across every other phase.
__device__ __forceinline__ int local_tid() { int t = (int)threadIdx.x; asm volatile("" : "+v"(t)); return t; }
template <typename T> __device__ __forceinline__ T* uni_ptr(T* p) {
    const unsigned long long v = (unsigned long long)p;
    const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)v);
    const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(v >> 32));
    return (T*)(((unsigned long long)hi << 32) | lo);
}
// Pointers read out of the phase table are generic to the compiler; every access goes through an
// explicit global-address-space pointer so it becomes a global_* instruction.  (A flat access counts
// on the LDS counter too, and a wait for an LDS read would then also wait for every weight load in
// flight.)
#define GPTRS_GLOBAL __attribute__((address_space(1)))
#define GPTRS_LDS __attribute__((address_space(3)))
template <typename T> __device__ __forceinline__ const GPTRS_GLOBAL T* as_global(const T* p) { return (const GPTRS_GLOBAL T*)p; }
template <typename T> __device__ __forceinline__ GPTRS_GLOBAL T* as_global(T* p) { return (GPTRS_GLOBAL T*)p; }
template <typename T> __device__ __forceinline__ T gload(const T* p) { return *as_global(p); }   // scalar T
template <typename T> __device__ __forceinline__ void gstore(T* p, const T& v) { *as_global(p) = v; }
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint2 gload2(const void* p) { const u32x2 v = *(const GPTRS_GLOBAL u32x2*)p; return make_uint2(v.x, v.y); }
__device__ __forceinline__ uint4 gload4(const void* p) { const u32x4 v = *(const GPTRS_GLOBAL u32x4*)p; return make_uint4(v.x, v.y, v.z, v.w); }
__device__ __forceinline__ void gstore4(void* p, const uint4& v) { u32x4 w; w.x = v.x; w.y = v.y; w.z = v.z; w.w = v.w; *(GPTRS_GLOBAL u32x4*)p = w; }
// agent-scope accesses: coherent across the XCDs' L2s without cache maintenance
__device__ __forceinline__ unsigned long long cload8(const void* p) {
    return __hip_atomic_load(as_global((const unsigned long long*)p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned cload4(const void* p) {
    return __hip_atomic_load(as_global((const unsigned*)p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void cstore8(void* p, unsigned long long v) {
    __hip_atomic_store(as_global((unsigned long long*)p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void cstore4(void* p, unsigned v) {
    __hip_atomic_store(as_global((unsigned*)p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// bf16 rounding with the hardware converter (v_cvt_pk_bf16_f32, round to nearest even): the staging of a
// normalised row runs these on every wave of the workgroup at once, where each instruction counts three times
// on the SIMD that holds three waves
__device__ __forceinline__ unsigned pack_hw(float lo, float hi) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    f32x2_t f;
    f.x = lo; f.y = hi;
    return __builtin_bit_cast(unsigned, __builtin_convertvector(f, bf16x2));
}
__device__ __forceinline__ float rbf(float v) { return bf16lo(pack_hw(v, 0.f)); }
template <typename P> __device__ __forceinline__ int lds_ld(P p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP); }
template <typename P> __device__ __forceinline__ void lds_st(P p, int v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP); }
#define GPTRS_LDS_RELEASE() __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local")
#define GPTRS_LDS_ACQUIRE() __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local")

struct alignas(16) Shared {
    float red[NSLOT][NWS][16];
    float epi_bias[EPI_MAX];
    float epi_res[EPI_MAX];
    // int8: [0, EPI_MAX) scale of each owned output column (gate of a SwiGLU pair), [EPI_MAX, 2 EPI_MAX) the pair's
    // up column.  (int4 group scales are staged behind the activations, see stage_block.)
    float epi_s[2 * EPI_MAX];
    float ssq[32];   // per-wave sums of the norm statistics (LayerNorm takes two rounds: [0, 16) and [16, 32))
    int red_cnt[NSLOT];
    int go, consumed, abort, pad;
};

// The table of phases is read-only for the whole launch: reading it through the constant address space lets the
// compiler use scalar loads (uniform addresses), which do not queue behind a wave's vector memory traffic.
#define GPTRS_CONST __attribute__((address_space(4)))
typedef const GPTRS_CONST ChainPhase* PhaseTable;
static_assert(sizeof(Shared) + (size_t)kChainMaxXsWords * 4 + (size_t)RING_MIN * SLOT_BYTES <= (size_t)LDS_BYTES, "the largest launch fits a CU's LDS");
constexpr int kPhaseDwords = (int)(sizeof(ChainPhase) / 4);
static_assert(kPhaseDwords <= 64, "one lane of the control wave per dword of a phase descriptor");

// Workgroup barrier that waits for this wave's LDS traffic only: the weight loads in flight stay in flight.
__device__ __forceinline__ void wg_barrier() {
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
}

// Uniform copy (scalar registers) of the descriptor fields that the staging and the epilogue read.  The compute waves
// fill it with scalar loads from the table before they wait for the phase to open; the control wave reads the table with
// one vector load (a lane per dword) before it waits for the grid barrier and picks the fields out of the lanes.  Either
// way nothing is fetched between the barrier and the first use.
struct PhaseRegs {
    int K, N, Kw, ntiles, upb, units, lds_bytes, flags, wfmt;
    float inv_n, eps;
    const void *x, *gamma, *beta, *bias, *residual, *wscale, *wscale2;
    void* y;
};
// (F32: the launch has f32 phases; only those read the LayerNorm offsets, and a register pair that nobody reads is not kept)
template <bool F32>
__device__ __forceinline__ void regs_from_table(PhaseRegs& R, const GPTRS_CONST ChainPhase* D) {
    R.K = uni(D->K); R.N = uni(D->N); R.Kw = uni(D->Kw); R.ntiles = uni(D->ntiles); R.upb = uni(D->upb); R.units = uni(D->units);
    R.lds_bytes = uni(D->lds_bytes); R.flags = uni(D->flags); R.wfmt = uni(D->wfmt);
    R.inv_n = __int_as_float(uni(__float_as_int(D->inv_n))); R.eps = __int_as_float(uni(__float_as_int(D->eps)));
    R.x = uni_ptr(D->x); R.gamma = uni_ptr(D->gamma); R.beta = F32 ? uni_ptr(D->beta) : nullptr; R.bias = uni_ptr(D->bias); R.residual = uni_ptr(D->residual);
    R.wscale = uni_ptr(D->wscale); R.wscale2 = uni_ptr(D->wscale2); R.y = uni_ptr(D->y);
}
#define GPTRS_PD_INT(field) __builtin_amdgcn_readlane(pd, (int)(offsetof(ChainPhase, field) / 4))
#define GPTRS_PD_PTR(field) ((const void*)(((unsigned long long)(unsigned)__builtin_amdgcn_readlane(pd, (int)(offsetof(ChainPhase, field) / 4) + 1) << 32) | \
                                          (unsigned)__builtin_amdgcn_readlane(pd, (int)(offsetof(ChainPhase, field) / 4))))
template <bool F32>
__device__ __forceinline__ void regs_from_lanes(PhaseRegs& R, int pd) {   // pd: dword `lane` of the descriptor
    R.K = GPTRS_PD_INT(K); R.N = GPTRS_PD_INT(N); R.Kw = GPTRS_PD_INT(Kw); R.ntiles = GPTRS_PD_INT(ntiles); R.upb = GPTRS_PD_INT(upb);
    R.units = GPTRS_PD_INT(units); R.lds_bytes = GPTRS_PD_INT(lds_bytes); R.flags = GPTRS_PD_INT(flags); R.wfmt = GPTRS_PD_INT(wfmt);
    R.inv_n = __int_as_float(GPTRS_PD_INT(inv_n)); R.eps = __int_as_float(GPTRS_PD_INT(eps));
    R.x = GPTRS_PD_PTR(x); R.gamma = GPTRS_PD_PTR(gamma); R.beta = F32 ? GPTRS_PD_PTR(beta) : nullptr; R.bias = GPTRS_PD_PTR(bias); R.residual = GPTRS_PD_PTR(residual);
    R.wscale = GPTRS_PD_PTR(wscale); R.wscale2 = GPTRS_PD_PTR(wscale2); R.y = const_cast<void*>(GPTRS_PD_PTR(y));
}

// ---------------------------------------------------------------------------- staging (all waves)
// xs[j] = (x[2j], x[2j+1]) as a bf16 pair, zero beyond K; with norm: the value the stand-alone
// RMSNorm kernels store, ((x * inv_rms) * gamma) -> bf16 (normalization.rs:183-217).
template <int FMT>
__device__ __forceinline__ void stage_block(const PhaseRegs& P, unsigned* xs, float* ssq) {
    const int t = local_tid(), lane = t & 63, wave = uni(t >> 6);
    const int K = P.K;
    const int n = K / 4;                     // 8-byte items holding data (K % 4 == 0)
    const int npad = P.lds_bytes >> 3;  // items to write: the words of every lane read zeros beyond K
    const char* x = (const char*)P.x;
    // int4: the group scales of this workgroup's tiles, one contiguous range of the tile-ordered copy
    // sc[tile][group][4] (bf16, 8 bytes per entry), go behind the activations; the first round of
    // loads is in flight while the activations are staged
    constexpr int SB = 8;
    int sc_n = 0;
    const uint2* sc_src = nullptr;
    uint2* sc_dst = reinterpret_cast<uint2*>(xs + 2 * npad);
    uint2 sv[SB];
    if (FMT == kChainW4) {   // (every linear phase of a launch has the kernel's weight format)
        const int G = P.Kw >> 4, upb = P.upb;
        const int t0 = (int)blockIdx.x * upb * TP, t1 = min(min(t0 + upb * TP, P.units * TP), P.ntiles);
        sc_n = max(t1 - t0, 0) * G;
        sc_src = (const uint2*)P.wscale + (long)t0 * G;
#pragma unroll
        for (int u = 0; u < SB; ++u) {
            const int i = u * NT + t;
            sv[u] = i < sc_n ? gload2(sc_src + i) : make_uint2(0u, 0u);
        }
    }
    if ((P.flags & (kChainNorm | kChainXF32)) == (kChainNorm | kChainXF32)) {
        // f32 row and gains (a bf16 model whose residual stream is f32): the f32 norm, rounded to bf16 once
        constexpr int MF = MAXI / 2;   // 16-byte items per thread: K <= 4 * MF * NT
        const char* g = (const char*)P.gamma;
        uint4 v[MF], gg[MF];
#pragma unroll
        for (int u = 0; u < MF; ++u) {
            const int i = u * NT + t;
            v[u] = make_uint4(0u, 0u, 0u, 0u);
            gg[u] = make_uint4(0u, 0u, 0u, 0u);
            if (u * NT < n && i < n) {
                const unsigned long long a = cload8(x + 16 * (size_t)i), b = cload8(x + 16 * (size_t)i + 8);
                v[u] = make_uint4((unsigned)a, (unsigned)(a >> 32), (unsigned)b, (unsigned)(b >> 32));
                gg[u] = gload4(g + 16 * (size_t)i);
            }
        }
        float q = 0.f;
#pragma unroll
        for (int u = 0; u < MF; ++u) {
            if (u * NT < n) {
                const float a = __uint_as_float(v[u].x), b = __uint_as_float(v[u].y), c = __uint_as_float(v[u].z), d = __uint_as_float(v[u].w);
                q += a * a; q += b * b; q += c * c; q += d * d;
            }
        }
        const float ws = wave_sum(q);
        if (lane == 0) ssq[wave] = ws;
        wg_barrier();
        float tot = 0.f;
#pragma unroll
        for (int w = 0; w < NT / 64; ++w) tot += ssq[w];
        const float inv = 1.0f / sqrtf(tot * P.inv_n + P.eps);
#pragma unroll
        for (int u = 0; u < MF; ++u) {
            const int i = u * NT + t;
            if (u * NT < npad && i < npad) {
                const unsigned o0 = pack_hw((__uint_as_float(v[u].x) * inv) * __uint_as_float(gg[u].x),
                                            (__uint_as_float(v[u].y) * inv) * __uint_as_float(gg[u].y));
                const unsigned o1 = pack_hw((__uint_as_float(v[u].z) * inv) * __uint_as_float(gg[u].z),
                                            (__uint_as_float(v[u].w) * inv) * __uint_as_float(gg[u].w));
                *reinterpret_cast<uint2*>(&xs[2 * i]) = make_uint2(o0, o1);
            }
        }
    } else if (P.flags & kChainNorm) {
        const uint2* g = (const uint2*)P.gamma;
        unsigned long long v[MAXI];
        uint2 gg[MAXI];
#pragma unroll
        for (int u = 0; u < MAXI; ++u) {
            const int i = u * NT + t;
            v[u] = 0ull;
            gg[u] = make_uint2(0u, 0u);
            if (u * NT < n && i < n) {
                v[u] = cload8(x + 8 * (size_t)i);
                gg[u] = gload2(g + i);
            }
        }
        // rounds beyond the row (wave-uniform test) are skipped: a short row must not pay for MAXI of them
        float q = 0.f;
#pragma unroll
        for (int u = 0; u < MAXI; ++u) {
            if (u * NT < n) {
                const unsigned lo = (unsigned)v[u], hi = (unsigned)(v[u] >> 32);
                const float a = bf16lo(lo), b = bf16hi(lo), c = bf16lo(hi), d = bf16hi(hi);
                q += a * a; q += b * b; q += c * c; q += d * d;
            }
        }
        const float ws = wave_sum(q);
        if (lane == 0) ssq[wave] = ws;
        wg_barrier();
        float tot = 0.f;
#pragma unroll
        for (int w = 0; w < NT / 64; ++w) tot += ssq[w];
        const float inv = 1.0f / sqrtf(tot * P.inv_n + P.eps);
#pragma unroll
        for (int u = 0; u < MAXI; ++u) {
            const int i = u * NT + t;
            if (u * NT < npad && i < npad) {
                const unsigned lo = (unsigned)v[u], hi = (unsigned)(v[u] >> 32);
                // (x * inv) * gamma in f32, rounded to bf16 once: what the stand-alone RMSNorm kernels store
                const unsigned o0 = pack_hw((bf16lo(lo) * inv) * bf16lo(gg[u].x), (bf16hi(lo) * inv) * bf16hi(gg[u].x));
                const unsigned o1 = pack_hw((bf16lo(hi) * inv) * bf16lo(gg[u].y), (bf16hi(hi) * inv) * bf16hi(gg[u].y));
                *reinterpret_cast<uint2*>(&xs[2 * i]) = make_uint2(o0, o1);
            }
        }
    } else {
        for (int i0 = 0; i0 < npad; i0 += MAXI * NT) {
            unsigned long long v[MAXI];
#pragma unroll
            for (int u = 0; u < MAXI; ++u) {
                const int i = i0 + u * NT + t;
                v[u] = i < n ? cload8(x + 8 * (size_t)i) : 0ull;
            }
#pragma unroll
            for (int u = 0; u < MAXI; ++u) {
                const int i = i0 + u * NT + t;
                if (i < npad) *reinterpret_cast<uint2*>(&xs[2 * i]) = make_uint2((unsigned)v[u], (unsigned)(v[u] >> 32));
            }
        }
    }
    if (FMT == kChainW4 && sc_n > 0) {
#pragma unroll
        for (int u = 0; u < SB; ++u) {
            const int i = u * NT + t;
            if (i < sc_n) sc_dst[i] = sv[u];
        }
        for (int i0 = SB * NT; i0 < sc_n; i0 += SB * NT) {
#pragma unroll
            for (int u = 0; u < SB; ++u) {
                const int i = i0 + u * NT + t;
                sv[u] = i < sc_n ? gload2(sc_src + i) : make_uint2(0u, 0u);
            }
#pragma unroll
            for (int u = 0; u < SB; ++u) {
                const int i = i0 + u * NT + t;
                if (i < sc_n) sc_dst[i] = sv[u];
            }
        }
    }
    wg_barrier();
}


// f32 phases (kChainW32): xs[j] = x[j] as f32, zero beyond K; with norm: LayerNorm as the stand-alone kernel computes it,
// ((x - mean) * inv_std) * gamma + beta with the mean and the variance of the centred row taken in two rounds
// (normalization.rs:36-120).
__device__ __forceinline__ void stage_block_f32(const PhaseRegs& P, unsigned* xs, float* ssq) {
    const int t = local_tid(), lane = t & 63, wave = uni(t >> 6);
    const int n = P.K / 4;                // 16-byte items holding data (K % 4 == 0)
    const int npad = P.lds_bytes >> 4;    // items the readers see
    const char* x = (const char*)P.x;
    constexpr int MF = MAXI / 2;          // items per thread: K <= 4 * MF * NT
    const bool norm = P.flags & kChainNorm;
    uint4 v[MF], gg[MF], bb[MF];
#pragma unroll
    for (int u = 0; u < MF; ++u) {
        const int i = u * NT + t;
        v[u] = make_uint4(0u, 0u, 0u, 0u);
        gg[u] = make_uint4(0u, 0u, 0u, 0u);
        bb[u] = make_uint4(0u, 0u, 0u, 0u);
        if (u * NT < n && i < n) {
            const unsigned long long a = cload8(x + 16 * (size_t)i), b = cload8(x + 16 * (size_t)i + 8);
            v[u] = make_uint4((unsigned)a, (unsigned)(a >> 32), (unsigned)b, (unsigned)(b >> 32));
            if (norm) {
                gg[u] = gload4((const char*)P.gamma + 16 * (size_t)i);
                bb[u] = gload4((const char*)P.beta + 16 * (size_t)i);
            }
        }
    }
    if (norm) {
        float s = 0.f;
#pragma unroll
        for (int u = 0; u < MF; ++u)
            if (u * NT < n) { s += __uint_as_float(v[u].x); s += __uint_as_float(v[u].y); s += __uint_as_float(v[u].z); s += __uint_as_float(v[u].w); }
        const float ws = wave_sum(s);
        if (lane == 0) ssq[wave] = ws;
        wg_barrier();
        float tot = 0.f;
#pragma unroll
        for (int w = 0; w < NT / 64; ++w) tot += ssq[w];
        const float mean = tot * P.inv_n;
        float c[MF][4];
        float q = 0.f;
#pragma unroll
        for (int u = 0; u < MF; ++u) {
            const bool in = u * NT < n && u * NT + t < n;
            c[u][0] = in ? __uint_as_float(v[u].x) - mean : 0.f;
            c[u][1] = in ? __uint_as_float(v[u].y) - mean : 0.f;
            c[u][2] = in ? __uint_as_float(v[u].z) - mean : 0.f;
            c[u][3] = in ? __uint_as_float(v[u].w) - mean : 0.f;
            q += c[u][0] * c[u][0]; q += c[u][1] * c[u][1]; q += c[u][2] * c[u][2]; q += c[u][3] * c[u][3];
        }
        const float wq = wave_sum(q);
        if (lane == 0) ssq[16 + wave] = wq;
        wg_barrier();
        float var = 0.f;
#pragma unroll
        for (int w = 0; w < NT / 64; ++w) var += ssq[16 + w];
        const float inv_std = 1.0f / sqrtf(var * P.inv_n + P.eps);
#pragma unroll
        for (int u = 0; u < MF; ++u) {
            v[u].x = __float_as_uint((c[u][0] * inv_std) * __uint_as_float(gg[u].x) + __uint_as_float(bb[u].x));
            v[u].y = __float_as_uint((c[u][1] * inv_std) * __uint_as_float(gg[u].y) + __uint_as_float(bb[u].y));
            v[u].z = __float_as_uint((c[u][2] * inv_std) * __uint_as_float(gg[u].z) + __uint_as_float(bb[u].z));
            v[u].w = __float_as_uint((c[u][3] * inv_std) * __uint_as_float(gg[u].w) + __uint_as_float(bb[u].w));
        }
    }
#pragma unroll
    for (int u = 0; u < MF; ++u) {
        const int i = u * NT + t;
        if (u * NT < npad && i < npad) *reinterpret_cast<uint4*>(&xs[4 * i]) = i < n ? v[u] : make_uint4(0u, 0u, 0u, 0u);
    }
    wg_barrier();
}

// ---------------------------------------------------------------------------- decode attention
constexpr int NW = NT / 64;

__device__ __forceinline__ void unpack8(unsigned long long a, unsigned long long b, float (&o)[8]) {
    const unsigned a0 = (unsigned)a, a1 = (unsigned)(a >> 32), b0 = (unsigned)b, b1 = (unsigned)(b >> 32);
    o[0] = bf16lo(a0); o[1] = bf16hi(a0); o[2] = bf16lo(a1); o[3] = bf16hi(a1);
    o[4] = bf16lo(b0); o[5] = bf16hi(b0); o[6] = bf16lo(b1); o[7] = bf16hi(b1);
}
// 8 consecutive bf16: coherent (written earlier in this launch) / plain (older than the launch)
__device__ __forceinline__ void cload_bf16x8(const bf16_t* p, float (&o)[8]) { unpack8(cload8(p), cload8(p + 4), o); }
__device__ __forceinline__ void load_bf16x8(const bf16_t* p, float (&o)[8]) {
    const uint4 v = gload4(p);
    o[0] = bf16lo(v.x); o[1] = bf16hi(v.x); o[2] = bf16lo(v.y); o[3] = bf16hi(v.y);
    o[4] = bf16lo(v.z); o[5] = bf16hi(v.z); o[6] = bf16lo(v.w); o[7] = bf16hi(v.w);
}
// Rotate-half RoPE (ops/functional/rotary.rs:430-536) while loading dims [c0, c0+8) of one head of
// the packed projection: dims below `half` pair with dim+half, the next `half` dims with dim-half,
// the rest pass through; the result is rounded to bf16 like a stored post-RoPE row.
__device__ __forceinline__ void cload_roped(const bf16_t* head, int c0, int half, const bf16_t* cs, const bf16_t* sn, float (&out)[8]) {
    float own[8];
    cload_bf16x8(head + c0, own);
    if (cs == nullptr || c0 >= 2 * half) {
#pragma unroll
        for (int v = 0; v < 8; ++v) out[v] = own[v];
        return;
    }
    const bool first = c0 < half;
    float other[8], c[8], sv[8];
    cload_bf16x8(head + (first ? c0 + half : c0 - half), other);
    const int j0 = first ? c0 : c0 - half;
    load_bf16x8(cs + j0, c);
    load_bf16x8(sn + j0, sv);
#pragma unroll
    for (int v = 0; v < 8; ++v) out[v] = rbf(first ? own[v] * c[v] - other[v] * sv[v] : own[v] * c[v] + other[v] * sv[v]);
}
__device__ __forceinline__ long clampl(long v, long lo, long hi) { return v < lo ? lo : (v > hi ? hi : v); }

__device__ __forceinline__ void unpack_u4(const uint4& v, float (&o)[8]) {
    o[0] = bf16lo(v.x); o[1] = bf16hi(v.x); o[2] = bf16lo(v.y); o[3] = bf16hi(v.y);
    o[4] = bf16lo(v.z); o[5] = bf16hi(v.z); o[6] = bf16lo(v.w); o[7] = bf16hi(v.w);
}
// Waits inside the kernel are bounded by wall-clock time (wall_clock64 ticks at 100 MHz): the control wave's wait for the
// grid barrier by the launch's budget, the waits on it inside the workgroup by a multiple of that, so that the control
// wave is the one to give up and say why.
struct Patience {
    unsigned long long t0, ticks;
    unsigned spins;
    __device__ __forceinline__ Patience(unsigned long long budget) : t0(0), ticks(budget), spins(0) {}
    __device__ __forceinline__ bool spent() {   // call once per poll; reads the clock every 64th time
        if ((++spins & 63u) != 0) return false;
        const unsigned long long now = wall_clock64();
        if (t0 == 0) { t0 = now; return false; }
        return now - t0 > ticks;
    }
};
// compute waves wait here until the control wave has seen the grid barrier of `phase`
template <typename IP>
__device__ __forceinline__ bool wait_go(IP go, IP abort, int phase, unsigned long long budget) {
    Patience pat(8 * budget);
    while (uni(lds_ld(go)) < phase) {
        __builtin_amdgcn_s_sleep(1);
        if (uni(lds_ld(abort)) || pat.spent()) return false;
    }
    return true;
}

// exp through v_exp_f32 (2^x): softmax weights only, about one ulp, exp(-inf) = 0
__device__ __forceinline__ float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896f); }
// sum over the lpr (8, 16 or 32) consecutive lanes of a lane group, result in each of them
__device__ __forceinline__ float group_sum(float v, int lpr) {
    int x = __float_as_int(v);
#define GPTRS_DPP_ADD(ctrl) x = __float_as_int(__int_as_float(x) + __int_as_float(__builtin_amdgcn_update_dpp(0, x, (ctrl), 0xf, 0xf, false)))
    GPTRS_DPP_ADD(0xB1);    // quad_perm [1,0,3,2]
    GPTRS_DPP_ADD(0x4E);    // quad_perm [2,3,0,1]
    GPTRS_DPP_ADD(0x141);   // row_half_mirror: 8 lanes
    if (lpr >= 16) GPTRS_DPP_ADD(0x140);  // row_mirror: 16 lanes
#undef GPTRS_DPP_ADD
    float r = __int_as_float(x);
    if (lpr == 32) {
        const u32x2 sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(r), __float_as_uint(r), false, false);
        r = __uint_as_float(sw.x) + __uint_as_float(sw.y);
    }
    return r;
}
// the values of v held by this lane and by its partner lane ^ off (off = 8, 16 or 32), in an order
// that is the same for both partners of a pair up to a swap: for symmetric merges only
__device__ __forceinline__ void lane_pair(float v, int off, float& a, float& b) {
    if (off == 8) {
        a = v;
        b = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xf, 0xf, false));  // row_ror:8
    } else if (off == 16) {
        const u32x2 sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
        a = __uint_as_float(sw.x); b = __uint_as_float(sw.y);
    } else {
        const u32x2 sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
        a = __uint_as_float(sw.x); b = __uint_as_float(sw.y);
    }
}

// unit = kv head * nch + chunk.  Each of the 8 streaming waves serves ONE query head of the kv
// head's group (wave w: head w % G, position subset w / G of 8 / G), so a lane carries a single
// online-softmax state; a cache row (head_dim bf16) is read by head_dim/8 lanes, 16 bytes each, and
// the waves of different heads re-read the same rows out of the caches.  Cache rows older than
// this launch are requested BEFORE the grid barrier is awaited (they do not depend on the
// previous phase); only the query row and this step's K/V row are read after it.
__device__ bool attn_partial(GPTRS_LDS int* go, GPTRS_LDS int* abort, const ChainPhase& P, GPTRS_LDS float* lds, int unit, int phase,
                             unsigned long long budget) {
    constexpr int PP = 5;   // positions per lane group requested ahead of the barrier (32 chunks x 8 lane groups x 5 = 1280 positions)
    const int t = local_tid(), lane = t & 63, wave = uni(t >> 6);
    const bool control = wave == NWS;
    const int dh = P.head_dim, n_q = P.n_q, n_kv = P.n_kv, nch = P.nch, half = P.rot_half;
    const int G = n_q / n_kv, nparts = NWS / G;
    const long cap = P.capacity;
    const int lpr = dh >> 3, rpw = 64 / lpr, sub = lane / lpr, li = lane % lpr;
    const int g = wave % G, part = wave / G;
    const int stride = nparts * rpw, sid = part * rpw + sub;   // position slots of this head's waves
    const int kvh = unit / nch, c = unit - kvh * nch;
    const bf16_t* qkv = (const bf16_t*)P.x;
    bf16_t* kc = (bf16_t*)P.k_cache;
    bf16_t* vc = (bf16_t*)P.v_cache;
    const bf16_t* cs = (const bf16_t*)P.cos;
    const bf16_t* sn = (const bf16_t*)P.sin;
    const long qpos = clampl(uni(gload(P.query_start)), 0, cap - 1);       // DynamicSlice clamp (cpu.rs:804-820)
    const long upd = clampl(uni(gload(P.update_starts + 1)), 0, cap - 1);  // DynamicUpdateSlice clamp
    const float scale = P.scale;
    const long L = qpos + 1, CL = (L + nch - 1) / nch;
    const long p0 = c * CL, p1 = min(L, p0 + CL);
    const int owner = (int)min(upd / CL, (long)nch - 1);
    const bf16_t* knew = qkv + (long)n_q * dh + (long)kvh * dh;
    const bf16_t* vnew = qkv + (long)(n_q + n_kv) * dh + (long)kvh * dh;
    const int c0 = li * 8;
    uint4 kraw[PP], vraw[PP];
#pragma unroll
    for (int j = 0; j < PP; ++j) {
        const long p = p0 + sid + (long)j * stride;
        if (!control && p < p1 && p != upd) {
            const long row = ((long)kvh * cap + p) * dh + c0;
            kraw[j] = gload4(kc + row);
            vraw[j] = gload4(vc + row);
        } else {
            kraw[j] = make_uint4(0, 0, 0, 0);
            vraw[j] = make_uint4(0, 0, 0, 0);
        }
    }
    if (!control && !wait_go(go, abort, phase, budget)) return false;

    float m = -INFINITY, l = 0.f, o[8];
#pragma unroll
    for (int v = 0; v < 8; ++v) o[v] = 0.f;
    if (!control) {
        // the wave's query head (RoPE applied on the fly) and, in the first lane group of each head's
        // first wave of the workgroup that owns position `upd`, this step's K/V row: all requested
        // before any is consumed
        const bool rot = cs != nullptr && c0 < 2 * half;
        const bool first = c0 < half;
        const int j0 = first ? c0 : c0 - half, co = first ? c0 + half : c0 - half;
        float cosv[8], sinv[8];
        if (rot) { load_bf16x8(cs + j0, cosv); load_bf16x8(sn + j0, sinv); }
        const bf16_t* head = qkv + (long)(kvh * G + g) * dh;
        unsigned long long qa[2], qb[2] = {0ull, 0ull};
        qa[0] = cload8(head + c0); qa[1] = cload8(head + c0 + 4);
        if (rot) { qb[0] = cload8(head + co); qb[1] = cload8(head + co + 4); }
        const bool fresh = c == owner && sid == 0;           // this lane group handles the new row
        unsigned long long ka[2] = {0ull, 0ull}, kb[2] = {0ull, 0ull}, va[2] = {0ull, 0ull};
        if (fresh) {
            ka[0] = cload8(knew + c0); ka[1] = cload8(knew + c0 + 4);
            if (rot) { kb[0] = cload8(knew + co); kb[1] = cload8(knew + co + 4); }
            va[0] = cload8(vnew + c0); va[1] = cload8(vnew + c0 + 4);
        }
        auto rope = [&](const unsigned long long (&own2)[2], const unsigned long long (&oth2)[2], float (&out)[8]) {
            float own[8], other[8];
            unpack8(own2[0], own2[1], own);
            if (!rot) {
#pragma unroll
                for (int v = 0; v < 8; ++v) out[v] = own[v];
                return;
            }
            unpack8(oth2[0], oth2[1], other);
#pragma unroll
            for (int v = 0; v < 8; ++v)
                out[v] = rbf(first ? own[v] * cosv[v] - other[v] * sinv[v] : own[v] * cosv[v] + other[v] * sinv[v]);
        };
        float qf[8];
        rope(qa, qb, qf);

        auto visit = [&](const float (&kf)[8], const float (&vf)[8]) {
            float sc = 0.f;
#pragma unroll
            for (int v = 0; v < 8; ++v) sc += qf[v] * kf[v];
            sc = group_sum(sc, lpr) * scale;
            const float mn = fmaxf(m, sc);
            const float corr = fast_exp(m - mn);
            const float pe = fast_exp(sc - mn);
            l = l * corr + pe;
#pragma unroll
            for (int v = 0; v < 8; ++v) o[v] = o[v] * corr + pe * vf[v];
            m = mn;
        };
#pragma unroll
        for (int j = 0; j < PP; ++j) {
            const long p = p0 + sid + (long)j * stride;
            if (p < p1 && p != upd) {
                float kf[8], vf[8];
                unpack_u4(kraw[j], kf);
                unpack_u4(vraw[j], vf);
                visit(kf, vf);
            }
        }
        for (long p = p0 + sid + (long)PP * stride; p < p1; p += stride) {
            if (p == upd) continue;
            float kf[8], vf[8];
            const long row = ((long)kvh * cap + p) * dh + c0;
            load_bf16x8(kc + row, kf);
            load_bf16x8(vc + row, vf);
            visit(kf, vf);
        }
        if (fresh) {   // this step's row: attended to when in range; appended once (by head 0's wave)
            float kf[8], vf[8];
            rope(ka, kb, kf);
            unpack8(va[0], va[1], vf);
            if (g == 0) {
                const long row = ((long)kvh * cap + upd) * dh + c0;
                gstore4(kc + row, make_uint4(pack_bf16x2(kf[0], kf[1]), pack_bf16x2(kf[2], kf[3]), pack_bf16x2(kf[4], kf[5]), pack_bf16x2(kf[6], kf[7])));
                gstore4(vc + row, make_uint4((unsigned)va[0], (unsigned)(va[0] >> 32), (unsigned)va[1], (unsigned)(va[1] >> 32)));
            }
            if (upd >= p0 && upd < p1) visit(kf, vf);
        }
        // merge the lane groups of this wave
        for (int off = lpr; off < 64; off <<= 1) {
            float ma, mb, la, lb;
            lane_pair(m, off, ma, mb);
            lane_pair(l, off, la, lb);
            const float mn = fmaxf(ma, mb);
            const float ca = mn == -INFINITY ? 0.f : fast_exp(ma - mn);
            const float cb = mn == -INFINITY ? 0.f : fast_exp(mb - mn);
            l = la * ca + lb * cb;
#pragma unroll
            for (int v = 0; v < 8; ++v) {
                float oa, ob;
                lane_pair(o[v], off, oa, ob);
                o[v] = oa * ca + ob * cb;
            }
            m = mn;
        }
    }
    // merge the waves of each head through LDS and leave one record per query head
    GPTRS_LDS float* sm = lds;
    GPTRS_LDS float* sl = lds + NWS;
    GPTRS_LDS float* so = lds + 2 * NWS;
    if (!control && sub == 0) {
        if (li == 0) { sm[wave] = m; sl[wave] = l; }
#pragma unroll
        for (int v = 0; v < 8; ++v) so[wave * dh + c0 + v] = o[v];
    }
    wg_barrier();
    float* partp = P.part;
    const bool final = P.flags & kChainAttnFinal;
    for (int idx = t; idx < G * dh; idx += NT) {
        const int gg = idx / dh, d = idx - gg * dh;
        float mn = -INFINITY;
        for (int w = gg; w < NWS; w += G) mn = fmaxf(mn, sm[w]);
        float Ls = 0.f, O = 0.f;
        if (mn != -INFINITY) {
            for (int w = gg; w < NWS; w += G) {
                const float cw = fast_exp(sm[w] - mn);
                Ls += sl[w] * cw;
                O += so[w * dh + d] * cw;
            }
        }
        if (final) {
            // one chunk per kv head: its record is the whole softmax, and the context row is written here (what the merge of
            // a single record gives: O / L)
            __hip_atomic_store(as_global((unsigned short*)P.y + (long)(kvh * G + gg) * dh + d), (unsigned short)pack_bf16x2(O / Ls, 0.f),
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            continue;
        }
        float* rec = partp + ((long)(kvh * G + gg) * nch + c) * (dh + 2);
        if (d == 0) { cstore4(rec, __float_as_uint(mn)); cstore4(rec + 1, __float_as_uint(Ls)); }
        cstore4(rec + 2 + d, __float_as_uint(O));
    }
    // every lane's stores (record words, the appended cache row) have left the CU before the control wave, which passes
    // this barrier last of all it executes here, reports the workgroup's arrival
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    wg_barrier();
    return true;
}

// unit = query head: softmax-merge of its nch chunk records into the context row.  Thread
// (sg, d2) reads the records of the chunks s = sg, sg + NW, ... for the dims (2 d2, 2 d2 + 1) in
// one round of loads and merges them locally; the NW subsets meet in LDS.
__device__ bool attn_combine(GPTRS_LDS int* go, GPTRS_LDS int* abort, const ChainPhase& P, GPTRS_LDS float* lds, int hq, int phase,
                             unsigned long long budget) {
    constexpr int MAXC = 8;   // chunks per thread: nch <= MAXC * NW
    const int t = local_tid(), wave = uni(t >> 6);
    const int dh = P.head_dim, nch = P.nch;
    if (wave != NWS && !wait_go(go, abort, phase, budget)) return false;
    const float* base = P.part + (long)hq * nch * (dh + 2);
    bf16_t* ctx = (bf16_t*)P.y;
    const int h2 = dh / 2;
    for (int d0 = 0; d0 < h2; d0 += 64) {
        const int d2 = d0 + (t & 63);
        const bool act = d2 < h2;
        unsigned long long ml[MAXC], ov[MAXC];
#pragma unroll
        for (int u = 0; u < MAXC; ++u) {
            const int s = wave + u * NW;
            const bool ok = act && s < nch;
            ml[u] = ok ? cload8(base + (long)s * (dh + 2)) : 0ull;
            ov[u] = ok ? cload8(base + (long)s * (dh + 2) + 2 + 2 * d2) : 0ull;
        }
        float mn = -INFINITY;
#pragma unroll
        for (int u = 0; u < MAXC; ++u)
            if (wave + u * NW < nch) mn = fmaxf(mn, __uint_as_float((unsigned)ml[u]));
        float Ls = 0.f, o0 = 0.f, o1 = 0.f;
#pragma unroll
        for (int u = 0; u < MAXC; ++u) {
            if (wave + u * NW < nch) {
                const float ms = __uint_as_float((unsigned)ml[u]);
                const float cw = ms == -INFINITY ? 0.f : fast_exp(ms - mn);
                Ls += __uint_as_float((unsigned)(ml[u] >> 32)) * cw;
                o0 += __uint_as_float((unsigned)ov[u]) * cw;
                o1 += __uint_as_float((unsigned)(ov[u] >> 32)) * cw;
            }
        }
        GPTRS_LDS f32x4* rec = (GPTRS_LDS f32x4*)lds;
        { f32x4 r4; r4.x = mn; r4.y = Ls; r4.z = o0; r4.w = o1; rec[wave * 64 + (t & 63)] = r4; }
        wg_barrier();
        if (wave == 0 && act) {
            float M = -INFINITY;
#pragma unroll
            for (int w = 0; w < NW; ++w) M = fmaxf(M, rec[w * 64 + t].x);
            float Lt = 0.f, a0 = 0.f, a1 = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                const f32x4 r = rec[w * 64 + t];
                const float cw = r.x == -INFINITY ? 0.f : fast_exp(r.x - M);
                Lt += r.y * cw; a0 += r.z * cw; a1 += r.w * cw;
            }
            cstore4(ctx + (long)hq * dh + 2 * d2, pack_bf16x2(a0 / Lt, a1 / Lt));
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the context words are out before the arrival is reported
        wg_barrier();
    }
    return true;
}

// The two attention phases once more with the element type as a parameter, instantiated for f32 rows and caches only (a
// lane's 8 values are then two 16-byte words; no RoPE): written this way the bf16 phases above lost a microsecond each
// to the compiler, so they keep their own text.
template <bool F32>
__device__ bool attn_partial_t(GPTRS_LDS int* go, GPTRS_LDS int* abort, const ChainPhase& P, GPTRS_LDS float* lds, int unit, int phase,
                             unsigned long long budget) {
    typedef typename std::conditional<F32, float, bf16_t>::type E;
    constexpr int PP = F32 ? 2 : 4;   // positions per lane group requested ahead of the barrier
    constexpr int RW = F32 ? 2 : 1;   // 16-byte words of a lane's 8 values
    const int t = local_tid(), lane = t & 63, wave = uni(t >> 6);
    const bool control = wave == NWS;
    const int dh = P.head_dim, n_q = P.n_q, n_kv = P.n_kv, nch = P.nch, half = P.rot_half;
    const int G = n_q / n_kv, nparts = NWS / G;
    const long cap = P.capacity;
    const int lpr = dh >> 3, rpw = 64 / lpr, sub = lane / lpr, li = lane % lpr;
    const int g = wave % G, part = wave / G;
    const int stride = nparts * rpw, sid = part * rpw + sub;   // position slots of this head's waves
    const int kvh = unit / nch, c = unit - kvh * nch;
    const E* qkv = (const E*)P.x;
    E* kc = (E*)P.k_cache;
    E* vc = (E*)P.v_cache;
    const bf16_t* cs = F32 ? nullptr : (const bf16_t*)P.cos;
    const bf16_t* sn = F32 ? nullptr : (const bf16_t*)P.sin;
    const long qpos = clampl(uni(gload(P.query_start)), 0, cap - 1);       // DynamicSlice clamp (cpu.rs:804-820)
    const long upd = clampl(uni(gload(P.update_starts + 1)), 0, cap - 1);  // DynamicUpdateSlice clamp
    const float scale = P.scale;
    const long L = qpos + 1, CL = (L + nch - 1) / nch;
    const long p0 = c * CL, p1 = min(L, p0 + CL);
    const int owner = (int)min(upd / CL, (long)nch - 1);
    const E* knew = qkv + (long)n_q * dh + (long)kvh * dh;
    const E* vnew = qkv + (long)(n_q + n_kv) * dh + (long)kvh * dh;
    const int c0 = li * 8;
    uint4 kraw[PP][RW], vraw[PP][RW];
#pragma unroll
    for (int j = 0; j < PP; ++j) {
        const long p = p0 + sid + (long)j * stride;
        const bool take = !control && p < p1 && p != upd;
        const long row = ((long)kvh * cap + p) * dh + c0;
#pragma unroll
        for (int r = 0; r < RW; ++r) {
            kraw[j][r] = take ? gload4(kc + row + 4 * r) : make_uint4(0, 0, 0, 0);
            vraw[j][r] = take ? gload4(vc + row + 4 * r) : make_uint4(0, 0, 0, 0);
        }
    }
    // a lane's 8 values of a row: unpacked from bf16 or taken as they are
    auto row_values = [&](const uint4 (&raw)[RW], float (&f)[8]) {
        if (F32) {
            f[0] = __uint_as_float(raw[0].x); f[1] = __uint_as_float(raw[0].y); f[2] = __uint_as_float(raw[0].z); f[3] = __uint_as_float(raw[0].w);
            f[4] = __uint_as_float(raw[RW - 1].x); f[5] = __uint_as_float(raw[RW - 1].y); f[6] = __uint_as_float(raw[RW - 1].z); f[7] = __uint_as_float(raw[RW - 1].w);
        } else {
            unpack_u4(raw[0], f);
        }
    };
    auto load_row = [&](const E* p, float (&f)[8]) {   // plain loads (cache rows older than this launch)
        uint4 raw[RW];
#pragma unroll
        for (int r = 0; r < RW; ++r) raw[r] = gload4(p + 4 * r);
        row_values(raw, f);
    };
    auto cload_row = [&](const E* p, unsigned long long (&w)[2 * RW]) {   // agent-scope loads (rows written by the phase before)
#pragma unroll
        for (int r = 0; r < 2 * RW; ++r) w[r] = cload8(p + (F32 ? 2 : 4) * r);
    };
    auto words_values = [&](const unsigned long long (&w)[2 * RW], float (&f)[8]) {
        if (F32) {
#pragma unroll
            for (int r = 0; r < 2 * RW; ++r) { f[(2 * r) & 7] = __uint_as_float((unsigned)w[r]); f[(2 * r + 1) & 7] = __uint_as_float((unsigned)(w[r] >> 32)); }
        } else {
            unpack8(w[0], w[1], f);
        }
    };
    if (!control && !wait_go(go, abort, phase, budget)) return false;

    float m = -INFINITY, l = 0.f, o[8];
#pragma unroll
    for (int v = 0; v < 8; ++v) o[v] = 0.f;
    if (!control) {
        // the wave's query head (RoPE applied on the fly) and, in the first lane group of each head's
        // first wave of the workgroup that owns position `upd`, this step's K/V row: all requested
        // before any is consumed
        const bool rot = cs != nullptr && c0 < 2 * half;
        const bool first = c0 < half;
        const int j0 = first ? c0 : c0 - half, co = first ? c0 + half : c0 - half;
        float cosv[8], sinv[8];
        if (rot) { load_bf16x8(cs + j0, cosv); load_bf16x8(sn + j0, sinv); }
        const E* head = qkv + (long)(kvh * G + g) * dh;
        unsigned long long qa[2 * RW], qb[2 * RW];
#pragma unroll
        for (int r = 0; r < 2 * RW; ++r) qb[r] = 0ull;
        cload_row(head + c0, qa);
        if (rot) cload_row(head + co, qb);
        const bool fresh = c == owner && sid == 0;           // this lane group handles the new row
        unsigned long long ka[2 * RW], kb[2 * RW], va[2 * RW];
#pragma unroll
        for (int r = 0; r < 2 * RW; ++r) { ka[r] = 0ull; kb[r] = 0ull; va[r] = 0ull; }
        if (fresh) {
            cload_row(knew + c0, ka);
            if (rot) cload_row(knew + co, kb);
            cload_row(vnew + c0, va);
        }
        auto rope = [&](const unsigned long long (&own2)[2 * RW], const unsigned long long (&oth2)[2 * RW], float (&out)[8]) {
            float own[8], other[8];
            words_values(own2, own);
            if (!rot) {
#pragma unroll
                for (int v = 0; v < 8; ++v) out[v] = own[v];
                return;
            }
            words_values(oth2, other);
#pragma unroll
            for (int v = 0; v < 8; ++v)
                out[v] = rbf(first ? own[v] * cosv[v] - other[v] * sinv[v] : own[v] * cosv[v] + other[v] * sinv[v]);
        };
        float qf[8];
        rope(qa, qb, qf);

        auto visit = [&](const float (&kf)[8], const float (&vf)[8]) {
            float sc = 0.f;
#pragma unroll
            for (int v = 0; v < 8; ++v) sc += qf[v] * kf[v];
            sc = group_sum(sc, lpr) * scale;
            const float mn = fmaxf(m, sc);
            const float corr = fast_exp(m - mn);
            const float pe = fast_exp(sc - mn);
            l = l * corr + pe;
#pragma unroll
            for (int v = 0; v < 8; ++v) o[v] = o[v] * corr + pe * vf[v];
            m = mn;
        };
#pragma unroll
        for (int j = 0; j < PP; ++j) {
            const long p = p0 + sid + (long)j * stride;
            if (p < p1 && p != upd) {
                float kf[8], vf[8];
                row_values(kraw[j], kf);
                row_values(vraw[j], vf);
                visit(kf, vf);
            }
        }
        for (long p = p0 + sid + (long)PP * stride; p < p1; p += stride) {
            if (p == upd) continue;
            float kf[8], vf[8];
            const long row = ((long)kvh * cap + p) * dh + c0;
            load_row(kc + row, kf);
            load_row(vc + row, vf);
            visit(kf, vf);
        }
        if (fresh) {   // this step's row: attended to when in range; appended once (by head 0's wave)
            float kf[8], vf[8];
            rope(ka, kb, kf);
            words_values(va, vf);
            if (g == 0) {
                const long row = ((long)kvh * cap + upd) * dh + c0;
                if (F32) {
#pragma unroll
                    for (int r = 0; r < RW; ++r) {
                        gstore4(kc + row + 4 * r, make_uint4((unsigned)ka[2 * r], (unsigned)(ka[2 * r] >> 32), (unsigned)ka[(2 * r + 1) % (2 * RW)], (unsigned)(ka[(2 * r + 1) % (2 * RW)] >> 32)));
                        gstore4(vc + row + 4 * r, make_uint4((unsigned)va[2 * r], (unsigned)(va[2 * r] >> 32), (unsigned)va[(2 * r + 1) % (2 * RW)], (unsigned)(va[(2 * r + 1) % (2 * RW)] >> 32)));
                    }
                } else {
                    gstore4(kc + row, make_uint4(pack_bf16x2(kf[0], kf[1]), pack_bf16x2(kf[2], kf[3]), pack_bf16x2(kf[4], kf[5]), pack_bf16x2(kf[6], kf[7])));
                    gstore4(vc + row, make_uint4((unsigned)va[0], (unsigned)(va[0] >> 32), (unsigned)va[1], (unsigned)(va[1] >> 32)));
                }
            }
            if (upd >= p0 && upd < p1) visit(kf, vf);
        }
        // merge the lane groups of this wave
        for (int off = lpr; off < 64; off <<= 1) {
            float ma, mb, la, lb;
            lane_pair(m, off, ma, mb);
            lane_pair(l, off, la, lb);
            const float mn = fmaxf(ma, mb);
            const float ca = mn == -INFINITY ? 0.f : fast_exp(ma - mn);
            const float cb = mn == -INFINITY ? 0.f : fast_exp(mb - mn);
            l = la * ca + lb * cb;
#pragma unroll
            for (int v = 0; v < 8; ++v) {
                float oa, ob;
                lane_pair(o[v], off, oa, ob);
                o[v] = oa * ca + ob * cb;
            }
            m = mn;
        }
    }
    // merge the waves of each head through LDS and leave one record per query head
    GPTRS_LDS float* sm = lds;
    GPTRS_LDS float* sl = lds + NWS;
    GPTRS_LDS float* so = lds + 2 * NWS;
    if (!control && sub == 0) {
        if (li == 0) { sm[wave] = m; sl[wave] = l; }
#pragma unroll
        for (int v = 0; v < 8; ++v) so[wave * dh + c0 + v] = o[v];
    }
    wg_barrier();
    float* partp = P.part;
    const bool final = P.flags & kChainAttnFinal;
    for (int idx = t; idx < G * dh; idx += NT) {
        const int gg = idx / dh, d = idx - gg * dh;
        float mn = -INFINITY;
        for (int w = gg; w < NWS; w += G) mn = fmaxf(mn, sm[w]);
        float Ls = 0.f, O = 0.f;
        if (mn != -INFINITY) {
            for (int w = gg; w < NWS; w += G) {
                const float cw = fast_exp(sm[w] - mn);
                Ls += sl[w] * cw;
                O += so[w * dh + d] * cw;
            }
        }
        if (final) {
            // one chunk per kv head: its record is the whole softmax, and the context row is written here (what the merge of
            // a single record gives: O / L)
            const long at = (long)(kvh * G + gg) * dh + d;
            if (F32) cstore4((float*)P.y + at, __float_as_uint(O / Ls));
            else __hip_atomic_store(as_global((unsigned short*)P.y + at), (unsigned short)pack_bf16x2(O / Ls, 0.f), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            continue;
        }
        float* rec = partp + ((long)(kvh * G + gg) * nch + c) * (dh + 2);
        if (d == 0) { cstore4(rec, __float_as_uint(mn)); cstore4(rec + 1, __float_as_uint(Ls)); }
        cstore4(rec + 2 + d, __float_as_uint(O));
    }
    // every lane's stores (record words, the appended cache row) have left the CU before the control wave, which passes
    // this barrier last of all it executes here, reports the workgroup's arrival
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    wg_barrier();
    return true;
}

// unit = query head: softmax-merge of its nch chunk records into the context row.  Thread
// (sg, d2) reads the records of the chunks s = sg, sg + NW, ... for the dims (2 d2, 2 d2 + 1) in
// one round of loads and merges them locally; the NW subsets meet in LDS.
template <bool F32>
__device__ bool attn_combine_t(GPTRS_LDS int* go, GPTRS_LDS int* abort, const ChainPhase& P, GPTRS_LDS float* lds, int hq, int phase,
                             unsigned long long budget) {
    constexpr int MAXC = 8;   // chunks per thread: nch <= MAXC * NW
    const int t = local_tid(), wave = uni(t >> 6);
    const int dh = P.head_dim, nch = P.nch;
    if (wave != NWS && !wait_go(go, abort, phase, budget)) return false;
    const float* base = P.part + (long)hq * nch * (dh + 2);
    bf16_t* ctx = (bf16_t*)P.y;
    const int h2 = dh / 2;
    for (int d0 = 0; d0 < h2; d0 += 64) {
        const int d2 = d0 + (t & 63);
        const bool act = d2 < h2;
        unsigned long long ml[MAXC], ov[MAXC];
#pragma unroll
        for (int u = 0; u < MAXC; ++u) {
            const int s = wave + u * NW;
            const bool ok = act && s < nch;
            ml[u] = ok ? cload8(base + (long)s * (dh + 2)) : 0ull;
            ov[u] = ok ? cload8(base + (long)s * (dh + 2) + 2 + 2 * d2) : 0ull;
        }
        float mn = -INFINITY;
#pragma unroll
        for (int u = 0; u < MAXC; ++u)
            if (wave + u * NW < nch) mn = fmaxf(mn, __uint_as_float((unsigned)ml[u]));
        float Ls = 0.f, o0 = 0.f, o1 = 0.f;
#pragma unroll
        for (int u = 0; u < MAXC; ++u) {
            if (wave + u * NW < nch) {
                const float ms = __uint_as_float((unsigned)ml[u]);
                const float cw = ms == -INFINITY ? 0.f : fast_exp(ms - mn);
                Ls += __uint_as_float((unsigned)(ml[u] >> 32)) * cw;
                o0 += __uint_as_float((unsigned)ov[u]) * cw;
                o1 += __uint_as_float((unsigned)(ov[u] >> 32)) * cw;
            }
        }
        GPTRS_LDS f32x4* rec = (GPTRS_LDS f32x4*)lds;
        { f32x4 r4; r4.x = mn; r4.y = Ls; r4.z = o0; r4.w = o1; rec[wave * 64 + (t & 63)] = r4; }
        wg_barrier();
        if (wave == 0 && act) {
            float M = -INFINITY;
#pragma unroll
            for (int w = 0; w < NW; ++w) M = fmaxf(M, rec[w * 64 + t].x);
            float Lt = 0.f, a0 = 0.f, a1 = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                const f32x4 r = rec[w * 64 + t];
                const float cw = r.x == -INFINITY ? 0.f : fast_exp(r.x - M);
                Lt += r.y * cw; a0 += r.z * cw; a1 += r.w * cw;
            }
            if (F32) cstore8((float*)P.y + (long)hq * dh + 2 * d2, (unsigned long long)__float_as_uint(a0 / Lt) | ((unsigned long long)__float_as_uint(a1 / Lt) << 32));
            else cstore4(ctx + (long)hq * dh + 2 * d2, pack_bf16x2(a0 / Lt, a1 / Lt));
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the context words are out before the arrival is reported
        wg_barrier();
    }
    return true;
}

// The 9 compute and control waves of the workgroup: the units blk, blk + grid, ... of an attention phase.  Kept out of
// line (its register needs must not leak into the compute loop); the LDS operands travel as explicit
// local-address-space pointers so their accesses stay ds_* instructions.
// The descriptor comes straight from the table in memory (scalar loads): the compute waves enter an attention phase, and
// request the cache rows it needs, before the control wave has seen the barrier and filled the LDS copy.
template <bool F32>
__device__ __forceinline__ bool run_attn_phase(const GPTRS_CONST ChainPhase* php, GPTRS_LDS float* lds, GPTRS_LDS int* go, GPTRS_LDS int* abort, int phase,
                                               unsigned long long budget) {
    ChainPhase P;
    {
        int* dst = reinterpret_cast<int*>(&P);
        const GPTRS_CONST int* src = (const GPTRS_CONST int*)php;
#pragma unroll
        for (int i = 0; i < kPhaseDwords; ++i) dst[i] = uni(src[i]);
    }
    const int kind = P.kind, units = P.units;
    for (int u = blockIdx.x; u < units; u += gridDim.x) {
        bool ok;
        if (F32) {
            if (kind == kChainAttnCombine) ok = attn_combine_t<true>(go, abort, P, lds, u, phase, budget);
            else ok = attn_partial_t<true>(go, abort, P, lds, u, phase, budget);
        } else {
            if (kind == kChainAttnCombine) ok = attn_combine(go, abort, P, lds, u, phase, budget);
            else ok = attn_partial(go, abort, P, lds, u, phase, budget);
        }
        if (!ok) return false;
    }
    return true;
}

// ---------------------------------------------------------------------------- control wave
__device__ __forceinline__ float finish(float v, int flags, float bias, float res) {
    if (flags & kChainBias) v += bias;                                           // tensor_ops.rs:42-56
    if (flags & kChainGelu) v = (v * 0.5f) * (erff(v / 1.41421354f) + 1.0f);     // activation.rs:96-113
    if (flags & kChainResidual) v += res;
    return v;
}

template <int FMT>
__device__ void control_wave(Shared& sh, unsigned* xs, const ChainPhase* phases, int nphases, unsigned* bar, int* abort_flag,
                             unsigned long long budget, int stall_phase) {
    PhaseTable table = (PhaseTable)phases;
    const int lane = threadIdx.x & 63;
    const int blk = blockIdx.x, per = gridDim.x / NC;
    const unsigned epoch = gload(bar + NC * 64);   // written by the previous launch, stable during this one
    int ucount = 0;
    for (int ph = 0; ph < nphases; ++ph) {
        // the phase's descriptor is requested before the wait for the barrier and lands in LDS after it, ahead of `go`
        const int pd = lane < kPhaseDwords ? gload(reinterpret_cast<const int*>(phases + ph) + lane) : 0;
        const GPTRS_CONST ChainPhase* D = table + ph;
        const int kind = uni(D->kind);
        const int upb = uni(D->upb), units = uni(D->units);
        const int u0 = kind == kChainLinear ? blk * upb : 0;
        const int u1 = kind == kChainLinear ? min(u0 + upb, units) : 0;
        if (ph > 0) {
            // stall_phase (a test hook, -1 otherwise): one arrival more than the grid can deliver is expected at that
            // phase, so this wait runs out of time and the give-up path below is taken
            const unsigned target = epoch + (unsigned)ph * per + (ph == stall_phase ? 1u : 0u);
            Patience pat(budget);
            bool ok = true;
            for (;;) {
                const unsigned v = lane < NC ? __hip_atomic_load(as_global(bar) + lane * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : target;
                if (__builtin_amdgcn_ballot_w64((int)(v - target) < 0) == 0) break;
                __builtin_amdgcn_s_sleep(1);
                if (pat.spent() || ((pat.spins & 63u) == 0 && __hip_atomic_load(as_global(abort_flag), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) { ok = false; break; }
            }
            if (!ok) {
                __hip_atomic_store(as_global(abort_flag), 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                lds_st(&sh.abort, 1);
                return;
            }
        }
        // the compute waves hold their own copy of the descriptor: the phase opens the moment the barrier is seen
        if (kind != kChainLinear) {
            if (blk < units) {
                if (lane == 0) lds_st(&sh.go, ph);
                run_attn_phase<FMT == kChainW32>(table + ph, (GPTRS_LDS float*)xs, (GPTRS_LDS int*)&sh.go, (GPTRS_LDS int*)&sh.abort, ph, budget);
            }
        } else if (u0 < u1) {
            if (lane == 0) lds_st(&sh.go, ph);
            PhaseRegs P;
            regs_from_lanes<FMT == kChainW32>(P, pd);
            const int flags = P.flags, ntiles = P.ntiles, N = P.N;
            const bool dual = flags & kChainDual;
            const int cpt = dual ? 2 : 4;              // output columns per tile
            const int col0 = u0 * TP * cpt;
            const int ncols = min((u1 - u0) * TP * cpt, EPI_MAX);
            // bias / residual / int8 scales of this workgroup's columns: the first round is requested before the
            // staging loads and written to LDS after the staging, so that its latency hides behind the staging
            // instead of holding up the workgroup's barrier inside it
            const unsigned* bias = (const unsigned*)P.bias;
            const char* resid = (const char*)P.residual;
            constexpr int wfmt = FMT;   // every linear phase of a launch has the kernel's weight format
            const unsigned* sg = wfmt == kChainW8 ? (const unsigned*)P.wscale : nullptr;
            const unsigned* su = wfmt == kChainW8 ? (const unsigned*)P.wscale2 : nullptr;
            const bool out_f32 = flags & kChainOutF32;   // y and the residual are f32
            unsigned long long e_rf = 0ull;              // two f32 residual values
            unsigned long long e_bf = 0ull;              // two f32 bias values (f32 phases)
            auto epi_load = [&](int i, unsigned& bw, unsigned& rw, unsigned& ga, unsigned& gb) {
                const int col = col0 + i;
                const bool in = i < ncols && col < N;
                if (wfmt == kChainW32) {
                    const u32x2 b2 = (bias && in) ? *(const GPTRS_GLOBAL u32x2*)((const char*)bias + 4 * (size_t)col) : u32x2{0u, 0u};
                    e_bf = (unsigned long long)b2.x | ((unsigned long long)b2.y << 32);
                    bw = 0u;
                } else
                bw = (bias && in) ? gload(bias + (col >> 1)) : 0u;
                if (out_f32) e_rf = (resid && in) ? cload8(resid + 4 * (size_t)col) : 0ull;
                rw = (resid && in && !out_f32) ? cload4(resid + 2 * (size_t)col) : 0u;
                ga = (sg && in) ? gload(sg + (col >> 1)) : 0u;
                gb = (su && in) ? gload(su + (col >> 1)) : 0u;
            };
            auto epi_store = [&](int i, unsigned bw, unsigned rw, unsigned ga, unsigned gb) {
                if (i >= ncols) return;
                if (bias || resid) {
                    *reinterpret_cast<float2*>(&sh.epi_bias[i]) = wfmt == kChainW32 ? make_float2(__uint_as_float((unsigned)e_bf), __uint_as_float((unsigned)(e_bf >> 32)))
                                                                                     : make_float2(bf16lo(bw), bf16hi(bw));
                    *reinterpret_cast<float2*>(&sh.epi_res[i]) = out_f32 ? make_float2(__uint_as_float((unsigned)e_rf), __uint_as_float((unsigned)(e_rf >> 32)))
                                                                          : make_float2(bf16lo(rw), bf16hi(rw));
                }
                if (sg) {
                    *reinterpret_cast<float2*>(&sh.epi_s[i]) = make_float2(bf16lo(ga), bf16hi(ga));
                    *reinterpret_cast<float2*>(&sh.epi_s[EPI_MAX + i]) = make_float2(bf16lo(gb), bf16hi(gb));
                }
            };
            const bool has_epi = bias || resid || sg;
            unsigned e_bw = 0u, e_rw = 0u, e_ga = 0u, e_gb = 0u;
            if (has_epi) epi_load(lane * 2, e_bw, e_rw, e_ga, e_gb);
            if (wfmt == kChainW32) stage_block_f32(P, xs, sh.ssq);
            else stage_block<FMT>(P, xs, sh.ssq);
            if (has_epi) {
                epi_store(lane * 2, e_bw, e_rw, e_ga, e_gb);
                for (int i = lane * 2 + 128; i < ncols; i += 128) {
                    epi_load(i, e_bw, e_rw, e_ga, e_gb);
                    epi_store(i, e_bw, e_rw, e_ga, e_gb);
                }
            }
            char* out = (char*)P.y;
            for (int u = u0; u < u1; ++u, ++ucount) {
                const int slot = ucount % NSLOT;
                Patience pat(8 * budget);
                while (lds_ld(&sh.red_cnt[slot]) < NWS) {
                    __builtin_amdgcn_s_sleep(1);
                    if (pat.spent()) {
                        lds_st(&sh.abort, 1);
                        __hip_atomic_store(as_global(abort_flag), 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        return;
                    }
                }
                GPTRS_LDS_ACQUIRE();
                float s[4] = {0.f, 0.f, 0.f, 0.f};
                if (lane < TP) {
#pragma unroll
                    for (int w = 0; w < NWS; ++w) {
                        const float4 v = *reinterpret_cast<const float4*>(&sh.red[slot][w][lane * 4]);
                        s[0] += v.x; s[1] += v.y; s[2] += v.z; s[3] += v.w;
                    }
                }
                __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "workgroup", "local");
                if (lane == 0) { lds_st(&sh.red_cnt[slot], 0); lds_st(&sh.consumed, ucount + 1); }
                const int tile = u * TP + lane;
                if (lane < TP && tile < ntiles) {
                    const int e = min(((u - u0) * TP + lane) * cpt, EPI_MAX - 4);
                    // the staged values of the tile's columns in one round of LDS reads, and only those the phase has
                    float sc[4] = {1.f, 1.f, 1.f, 1.f}, bi[4] = {0.f, 0.f, 0.f, 0.f}, re[4] = {0.f, 0.f, 0.f, 0.f};
                    if (wfmt == kChainW8) {
                        if (dual) {
                            const float2 a = *reinterpret_cast<const float2*>(&sh.epi_s[e]), b = *reinterpret_cast<const float2*>(&sh.epi_s[EPI_MAX + e]);
                            sc[0] = a.x; sc[1] = b.x; sc[2] = a.y; sc[3] = b.y;
                        } else {
                            const float4 a = *reinterpret_cast<const float4*>(&sh.epi_s[e]);
                            sc[0] = a.x; sc[1] = a.y; sc[2] = a.z; sc[3] = a.w;
                        }
                    }
                    if (flags & (kChainBias | kChainResidual)) {   // both arrays are staged when either is present
                        if (dual) {
                            const float2 b = *reinterpret_cast<const float2*>(&sh.epi_bias[e]), r = *reinterpret_cast<const float2*>(&sh.epi_res[e]);
                            bi[0] = b.x; bi[1] = b.y; re[0] = r.x; re[1] = r.y;
                        } else {
                            const float4 b = *reinterpret_cast<const float4*>(&sh.epi_bias[e]), r = *reinterpret_cast<const float4*>(&sh.epi_res[e]);
                            bi[0] = b.x; bi[1] = b.y; bi[2] = b.z; bi[3] = b.w;
                            re[0] = r.x; re[1] = r.y; re[2] = r.z; re[3] = r.w;
                        }
                    }
                    if (wfmt == kChainW8) {
#pragma unroll
                        for (int c = 0; c < 4; ++c) s[c] *= sc[c];
                    }
                    if (dual) {   // columns interleaved (gate, up, gate, up): activation.rs:141-162
                        const float a0 = finish((s[0] / (1.0f + expf(s[0] * -1.0f))) * s[1], flags, bi[0], re[0]);
                        const float a1 = finish((s[2] / (1.0f + expf(s[2] * -1.0f))) * s[3], flags, bi[1], re[1]);
                        cstore4(out + 2 * (size_t)(tile * 2), pack_hw(a0, a1));
                    } else {
                        float o[4];
#pragma unroll
                        for (int c = 0; c < 4; ++c) o[c] = finish(s[c], flags, bi[c], re[c]);
                        if (tile * 4 + 4 > N) {   // the last tile of a width that is not a multiple of 4: its real columns one by one
#pragma unroll
                            for (int c = 0; c < 4; ++c) {
                                if (tile * 4 + c >= N) continue;
                                if (out_f32) cstore4(out + 4 * (size_t)(tile * 4 + c), __float_as_uint(o[c]));
                                else __hip_atomic_store(as_global((unsigned short*)out + (size_t)(tile * 4 + c)), (unsigned short)pack_hw(o[c], 0.f), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            }
                        } else if (out_f32) {
                            cstore8(out + 4 * (size_t)(tile * 4), (unsigned long long)__float_as_uint(o[0]) | ((unsigned long long)__float_as_uint(o[1]) << 32));
                            cstore8(out + 4 * (size_t)(tile * 4) + 8, (unsigned long long)__float_as_uint(o[2]) | ((unsigned long long)__float_as_uint(o[3]) << 32));
                        } else {
                            cstore8(out + 2 * (size_t)(tile * 4), (unsigned long long)pack_hw(o[0], o[1]) | ((unsigned long long)pack_hw(o[2], o[3]) << 32));
                        }
                    }
                }
            }
        }
        // this workgroup's outputs have left the CU before it arrives at the barrier
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        asm volatile("" ::: "memory");
        if (lane == 0) __hip_atomic_fetch_add(as_global(bar) + (blk % NC) * 64, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    // every launch advances each counter by nphases * per: the next launch starts from there
    if (blk == 0 && lane == 0) gstore(bar + NC * 64, epoch + (unsigned)nphases * per);
}

// Sums each of a wave's 12 per-lane accumulators (3 tiles x 4 columns) over its 64 lanes as a
// reduce-scatter: exchanging half of the values with lane ^ 32 and then lane ^ 16 leaves every 16-lane row
// with 3 values already summed over 4 lanes, which 4 row-wide DPP steps finish: 30 cross-lane operations where
// 12 separate wave sums take 120.  Returns in lanes 16r + s (s < 3) the total of accumulator 3r + s, i.e.
// element 3r + s of acc[p][c] taken as acc[0][0..3], acc[1][0..3], acc[2][0..3].
__device__ __forceinline__ float reduce_unit(const float (&acc)[TP][4], int lane) {
    static_assert(TP == 3, "12 accumulators per lane");
    float v[12];
#pragma unroll
    for (int p = 0; p < TP; ++p)
#pragma unroll
        for (int c = 0; c < 4; ++c) v[p * 4 + c] = acc[p][c];
    float h[6];
#pragma unroll
    for (int k = 0; k < 6; ++k) {   // lanes < 32 keep values 0..5, lanes >= 32 values 6..11
        const u32x2 sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(v[k]), __float_as_uint(v[k + 6]), false, false);
        h[k] = __uint_as_float(sw.x) + __uint_as_float(sw.y);
    }
    float q[3];
#pragma unroll
    for (int k = 0; k < 3; ++k) {   // even rows keep values k, odd rows values k + 3 of their half
        const u32x2 sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(h[k]), __float_as_uint(h[k + 3]), false, false);
        q[k] = __uint_as_float(sw.x) + __uint_as_float(sw.y);
    }
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        int x = __float_as_int(q[k]);
#define GPTRS_DPP_ADD(ctrl) x = __float_as_int(__int_as_float(x) + __int_as_float(__builtin_amdgcn_update_dpp(0, x, (ctrl), 0xf, 0xf, false)))
        GPTRS_DPP_ADD(0xB1);    // quad_perm [1,0,3,2]
        GPTRS_DPP_ADD(0x4E);    // quad_perm [2,3,0,1]
        GPTRS_DPP_ADD(0x141);   // row_half_mirror
        GPTRS_DPP_ADD(0x140);   // row_mirror
#undef GPTRS_DPP_ADD
        q[k] = __int_as_float(x);
    }
    const int sidx = lane & 15;
    return sidx == 0 ? q[0] : (sidx == 1 ? q[1] : q[2]);
}

// ---------------------------------------------------------------------------- compute waves
// s_waitcnt that waits until at most 3 * steps vector memory operations of the wave are in flight (and for nothing else);
// the count is an immediate of the instruction
template <int N> __device__ __forceinline__ void wait_vm_imm() { __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14)); }
__device__ __forceinline__ void wait_vm_count(int n) {   // steps without loads in flight (padding, tiles that do not exist): rare
    switch (n) {
#define GPTRS_VM(k) case k: wait_vm_imm<k>(); break;
        GPTRS_VM(1) GPTRS_VM(2) GPTRS_VM(3) GPTRS_VM(4) GPTRS_VM(5) GPTRS_VM(6) GPTRS_VM(7) GPTRS_VM(8)
        GPTRS_VM(9) GPTRS_VM(10) GPTRS_VM(11) GPTRS_VM(12)
#undef GPTRS_VM
        default: wait_vm_imm<0>(); break;   // 0, and anything unexpected: wait for everything
    }
    static_assert(3 * (RING_MAX - 1) <= 12, "cases above");
}

template <int FMT, int RING_D>
__device__ void compute_waves(Shared& sh, const unsigned* xs, PhaseTable table, int nphases, const unsigned char* ring, unsigned long long budget) {
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int blk = blockIdx.x;
    constexpr int kpw = FMT == kChainW32 ? 1 : (FMT == kChainW16 ? 2 : (FMT == kChainW8 ? 4 : 8));
    constexpr unsigned STEP = NS * 16;   // bytes of a tile stream per j-step

    // ---- request side: the wave's next j-step to ask for, in the order the steps are consumed.  Everything but r_off is
    // uniform: a request costs one vector add and clamp, three scalar moves and three loads.
    int r_phase = -1, r_unit = 0, r_unit_end = 0, r_j = 0, r_wpt = 1, r_ntiles = 1;
    unsigned r_last = 0;              // byte offset of a tile stream's last weight word
    unsigned r_tile_bytes = 0;        // bytes of a tile stream
    unsigned long long r_w = 0, r_base[TP] = {0, 0, 0};   // tile streams of the unit
    unsigned r_off = 0;               // this lane's byte offset in a tile stream at step r_j
    const unsigned ring_lds = (unsigned)uni((int)((unsigned)(size_t)(GPTRS_LDS unsigned char*)ring + (unsigned)(wave * 1024)));
    const unsigned ring_end = ring_lds + RING_D * SLOT_BYTES;
    unsigned r_dst = ring_lds;        // LDS address of lane 0's word of tile 0 in the next slot to fill
    int inflight = 0;                 // j-steps requested and not yet read
    unsigned pend = 0u;               // bits 2i, 2i + 1: loads that the i-th oldest of them carries
    int loads = 0;                    // loads in flight
    int r_tiles = TP;                 // tiles of the unit that exist
    bool r_plain = false;             // the unit has all its tiles and its streams end with a j-step
    auto r_unit_setup = [&]() {
        // a phase's last tiles may not exist: nothing is fetched for them
        r_tiles = min(TP, r_ntiles - r_unit * TP);
        r_plain = r_tiles == TP && r_last + 16u == (unsigned)r_wpt * STEP;
#pragma unroll
        for (int p = 0; p < TP; ++p) r_base[p] = r_w + (unsigned long long)(unsigned)min(r_unit * TP + p, r_ntiles - 1) * r_tile_bytes;
        r_off = (unsigned)t * 16u;
        r_j = 0;
    };
    auto r_seek = [&]() -> bool {   // next linear phase in which this workgroup has units
        for (;;) {
            ++r_phase;
            if (r_phase >= nphases) return false;
            const GPTRS_CONST ChainPhase* D = table + r_phase;
            if (uni(D->kind) != kChainLinear) continue;
            const int upb = uni(D->upb);
            r_unit = blk * upb;
            r_unit_end = min(r_unit + upb, uni(D->units));
            if (r_unit >= r_unit_end) continue;
            r_wpt = uni(D->wpt);
            r_ntiles = uni(D->ntiles);
            r_tile_bytes = (unsigned)uni(D->Kw) * 16u;
            r_last = (unsigned)((uni(D->K) + kpw - 1) / kpw - 1) * 16u;
            r_w = (unsigned long long)uni_ptr(D->w);
            r_unit_setup();
            return true;
        }
    };
    bool r_more = r_seek();
    // Asks for one j-step: one load per tile of the unit that exists (three but for a phase's last unit), none when all of
    // the wave's words of the step are padding behind K (the reader counts such words as zeros, and sums of tiles that do
    // not exist are never stored); `pend` records how many loads each step in flight carries, two bits per step, oldest
    // first.  Every load that is issued fetches weights never fetched before, so all of them take the same way through
    // the memory system and return in the order of issue: a load that re-read words already in a cache was seen to
    // complete ahead of older ones, which a count of loads in flight cannot express.  Lanes behind K in a partly filled
    // wave issue nothing.
    auto request = [&]() {
        int cnt = TP;
        if (__builtin_expect(r_plain, 1)) {   // three tiles, no padding: nothing to decide
#pragma unroll
            for (int p = 0; p < TP; ++p)   // M0: LDS address of lane 0's word
                asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(r_off), "s"((unsigned long long)uni_ptr((const char*)r_base[p])), "s"((unsigned)uni((int)(r_dst + (unsigned)(p * NS * 16)))) : "memory", "m0");
        } else {
            const bool any = (unsigned)((r_j * NS + wave * 64) * 16) <= r_last;   // the wave's first word of the step holds weights
            cnt = any ? r_tiles : 0;
            if (any) {
                if (r_off <= r_last) {
#pragma unroll
                    for (int p = 0; p < TP; ++p)
                        if (p < r_tiles)
                            asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(r_off), "s"((unsigned long long)uni_ptr((const char*)r_base[p])), "s"((unsigned)uni((int)(r_dst + (unsigned)(p * NS * 16)))) : "memory", "m0");
                }
            }
        }
        pend |= (unsigned)cnt << (2 * inflight);
        loads += cnt;
        r_off += STEP;
        r_dst += SLOT_BYTES;
        if (r_dst == ring_end) r_dst = ring_lds;
        ++inflight;
        if (++r_j == r_wpt) {
            if (++r_unit < r_unit_end) r_unit_setup();
            else r_more = r_seek();
        }
    };
    for (int i = 0; i < RING_D && r_more; ++i) request();

    // ---- read side
    int c_phase = -1, c_unit = 0, c_unit_end = 0, c_j = 0, c_wpt = 1, c_sidx = 0, c_G = 0, c_soff = 0, c_Kv = 0, ucount = 0;
    int c_consumed = 0;   // units the control wave has taken, as last read
    constexpr int c_fmt = FMT;
    PhaseRegs R;
    // advance to this workgroup's next linear unit, taking part in attention phases on the way
    auto c_seek = [&]() -> bool {
        for (;;) {
            ++c_phase;
            if (c_phase >= nphases) return false;
            const GPTRS_CONST ChainPhase* D = table + c_phase;   // the fields that decide this workgroup's part, before the wait
            const int units = uni(D->units);
            if (uni(D->kind) != kChainLinear) {
                if (blk >= units) continue;
                if (!run_attn_phase<FMT == kChainW32>(table + c_phase, (GPTRS_LDS float*)xs, (GPTRS_LDS int*)&sh.go, (GPTRS_LDS int*)&sh.abort, c_phase,
                                    budget)) return false;
                continue;
            }
            const int upb = uni(D->upb);
            c_unit = blk * upb;
            c_unit_end = min(c_unit + upb, units);
            if (c_unit >= c_unit_end) continue;
            c_wpt = uni(D->wpt);
            c_G = uni(D->Kw) >> 4;
            c_Kv = (uni(D->K) + kpw - 1) / kpw;
            c_sidx = 0;   // int4: entry of the unit's first tile and group in the staged scales ...
            c_soff = uni(D->lds_bytes) >> 2;   // ... which sit behind the activations
            regs_from_table<FMT == kChainW32>(R, D);
            return true;   // (the caller waits for the phase to open and stages its input)
        }
    };

    float acc[TP][4];
#pragma unroll
    for (int p = 0; p < TP; ++p)
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[p][c] = 0.f;
    int slot = 0;
    const GPTRS_LDS u32x4* mine = (const GPTRS_LDS u32x4*)ring + t;   // this lane's word of tile 0 in slot 0

    // A request can hold its wave for a microsecond (the memory pipeline of a CU takes a limited number of requests, and one
    // beyond that waits for an older one to land), so the request that a read frees is made after the step's arithmetic
    // and, at the end of a unit, after the partial sums are handed over: nothing the workgroup waits for stands behind it.
    // phases (rare code: seek, attention, staging) around units around j-steps (the loop that has to be tight)
    bool alive = true;
    while (alive && c_seek()) {
      // Until the phase opens the wave has nothing to do, its ring is full, and whatever of it has landed cannot be used
      // yet: the memory system would idle through the barrier.  So the oldest steps that have landed move from the ring
      // into registers (`park`), and the slots they leave are asked to fetch further ahead: up to PARK more j-steps of
      // weights are on their way while the grid synchronises.  Parked steps are the phase's first ones and are read
      // back first; the registers are free again before the next phase is looked for.
      constexpr int PARKN = FMT == kChainW4 ? PARK_W4 : (FMT == kChainW8 ? PARK_W8 : PARK);   // (the int4 kernel stages its group scales through registers as well)
      u32x4 park[PARKN][TP];
      int n_parked = 0, park_rd = 0;
      {
        const int want = min(PARKN, min(c_wpt * (c_unit_end - c_unit), inflight));
#pragma unroll
        for (int i = 0; i < PARKN; ++i) {
            if (i < want && uni(lds_ld(&sh.go)) < c_phase) {
                const GPTRS_LDS u32x4* wp = mine + slot * (SLOT_BYTES / 16);
                // The wave has time, so it waits for everything it has in flight rather than for this step alone: the request
                // it makes below then meets an empty queue and returns at once, and the wave is back at the test of `go`
                // instead of held in the memory pipeline behind its own older requests when the phase opens.
                if (loads) wait_vm_imm<0>();
                pend = 0u;
                loads = 0;
                asm volatile("" ::: "memory");
#pragma unroll
                for (int p = 0; p < TP; ++p) park[i][p] = wp[p * NS];
                --inflight;
                if (++slot == RING_D) slot = 0;
                __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0): the words are in registers before their slot is asked to take new ones
                asm volatile("" ::: "memory");
                if (r_more) request();
                n_parked = i + 1;
            }
        }
      }
      if (!wait_go(&sh.go, &sh.abort, c_phase, budget)) break;
      if (FMT == kChainW32) stage_block_f32(R, const_cast<unsigned*>(xs), sh.ssq);
      else stage_block<FMT>(R, const_cast<unsigned*>(xs), sh.ssq);
      bool from_park = false;
      for (; c_unit < c_unit_end; ++c_unit) {
        for (c_j = 0; c_j < c_wpt; ++c_j) {
        u32x4 cur[TP];
        from_park = park_rd < n_parked;
        if (from_park) {
            switch (park_rd) {
#define GPTRS_PARK(k) case k: _Pragma("unroll") for (int p = 0; p < TP; ++p) cur[p] = park[k < PARKN ? k : 0][p]; break;
                GPTRS_PARK(0) GPTRS_PARK(1)
                default: _Pragma("unroll") for (int p = 0; p < TP; ++p) cur[p] = park[PARKN - 1][p]; break;
#undef GPTRS_PARK
            }
            static_assert(PARK >= 1 && PARK <= 3 && PARK_W4 >= 1 && PARK_W4 <= 3 && PARK_W8 >= 1 && PARK_W8 <= 3, "cases above");
            ++park_rd;
        } else {
        const GPTRS_LDS u32x4* wp = mine + slot * (SLOT_BYTES / 16);
        // the loads of this j-step are the oldest in flight: they have landed once no more than the younger ones remain
        {
            const int oldest = (int)(pend & 3u), younger = loads - oldest;
            if (oldest) {
                if (__builtin_expect(younger == 3 * (RING_D - 1), 1)) wait_vm_imm<3 * (RING_D - 1)>();
                else wait_vm_count(younger);
            }
            pend >>= 2;
            loads = younger;
        }
        asm volatile("" ::: "memory");
#pragma unroll
        for (int p = 0; p < TP; ++p) cur[p] = wp[p * NS];
        --inflight;
        if (++slot == RING_D) slot = 0;
        }
        if ((c_j + 1) * NS > c_Kv) {   // the stream's last step: lanes whose words are padding count as zeros
            if (c_j * NS + t >= c_Kv) {
#pragma unroll
                for (int p = 0; p < TP; ++p) { cur[p].x = 0u; cur[p].y = 0u; cur[p].z = 0u; cur[p].w = 0u; }
            }
        }
        // element reads go through scalars: __builtin_bit_cast applied directly to `vec.y` of an
        // ext-vector reads element 0 with this compiler
        if (c_fmt == kChainW16) {
            const bf16x2 xv = __builtin_bit_cast(bf16x2, xs[c_j * NS + t]);
#pragma unroll
            for (int p = 0; p < TP; ++p) {
                const unsigned q0 = cur[p].x, q1 = cur[p].y, q2 = cur[p].z, q3 = cur[p].w;
                acc[p][0] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, q0), xv, acc[p][0], false);
                acc[p][1] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, q1), xv, acc[p][1], false);
                acc[p][2] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, q2), xv, acc[p][2], false);
                acc[p][3] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, q3), xv, acc[p][3], false);
            }
        } else if (c_fmt == kChainW32) {
            const float xv = __uint_as_float(xs[c_j * NS + t]);
#pragma unroll
            for (int p = 0; p < TP; ++p) {
                const unsigned q0 = cur[p].x, q1 = cur[p].y, q2 = cur[p].z, q3 = cur[p].w;
                acc[p][0] = __builtin_fmaf(__uint_as_float(q0), xv, acc[p][0]);
                acc[p][1] = __builtin_fmaf(__uint_as_float(q1), xv, acc[p][1]);
                acc[p][2] = __builtin_fmaf(__uint_as_float(q2), xv, acc[p][2]);
                acc[p][3] = __builtin_fmaf(__uint_as_float(q3), xv, acc[p][3]);
            }
        } else if (c_fmt == kChainW8) {
            const u32x2 xw = *reinterpret_cast<const u32x2*>(&xs[2 * (c_j * NS + t)]);
            const unsigned xa = xw.x, xb = xw.y;
            const float x0 = bf16lo(xa), x1 = bf16hi(xa), x2 = bf16lo(xb), x3 = bf16hi(xb);
            const float corr = -128.0f * ((x0 + x1) + (x2 + x3));
#pragma unroll
            for (int p = 0; p < TP; ++p) {
                const unsigned q[4] = {cur[p].x, cur[p].y, cur[p].z, cur[p].w};
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    float a = acc[p][c] + corr;
                    a = __builtin_fmaf((float)(q[c] & 0xFFu), x0, a);
                    a = __builtin_fmaf((float)((q[c] >> 8) & 0xFFu), x1, a);
                    a = __builtin_fmaf((float)((q[c] >> 16) & 0xFFu), x2, a);
                    a = __builtin_fmaf((float)(q[c] >> 24), x3, a);
                    acc[p][c] = a;
                }
            }
        } else {
            const u32x4 xw = *reinterpret_cast<const u32x4*>(&xs[4 * (c_j * NS + t)]);
            const unsigned xa = xw.x, xb = xw.y, xc = xw.z, xd = xw.w;
            const float x0 = bf16lo(xa), x1 = bf16hi(xa), x2 = bf16lo(xb), x3 = bf16hi(xb);
            const float x4 = bf16lo(xc), x5 = bf16hi(xc), x6 = bf16lo(xd), x7 = bf16hi(xd);
            const float corr = -8.0f * (((x0 + x1) + (x2 + x3)) + ((x4 + x5) + (x6 + x7)));
#pragma unroll
            for (int p = 0; p < TP; ++p) {
                const unsigned q[4] = {cur[p].x, cur[p].y, cur[p].z, cur[p].w};
                const u32x2 sw = *reinterpret_cast<const u32x2*>(&xs[c_soff + 2 * (c_sidx + p * c_G + c_j * (NS / 16) + (t >> 4))]);
                const unsigned sa = sw.x, sb = sw.y;
                const float sc[4] = {bf16lo(sa), bf16hi(sa), bf16lo(sb), bf16hi(sb)};
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    // byte i of a column's dword: k = 2i in the low nibble, k = 2i + 1 in the high one
                    const unsigned lo = q[c] & 0x0F0F0F0Fu, hi = (q[c] >> 4) & 0x0F0F0F0Fu;
                    float a = corr;
                    a = __builtin_fmaf((float)(lo & 0xFFu), x0, a);
                    a = __builtin_fmaf((float)(hi & 0xFFu), x1, a);
                    a = __builtin_fmaf((float)((lo >> 8) & 0xFFu), x2, a);
                    a = __builtin_fmaf((float)((hi >> 8) & 0xFFu), x3, a);
                    a = __builtin_fmaf((float)((lo >> 16) & 0xFFu), x4, a);
                    a = __builtin_fmaf((float)((hi >> 16) & 0xFFu), x5, a);
                    a = __builtin_fmaf((float)(lo >> 24), x6, a);
                    a = __builtin_fmaf((float)(hi >> 24), x7, a);
                    acc[p][c] = __builtin_fmaf(sc[c], a, acc[p][c]);
                }
            }
        }
        if (!from_park && c_j + 1 < c_wpt && r_more) request();   // (the unit's last step: after the hand-over below; a parked step's slot was refilled when it was parked)
        }   // j-steps
        {
            const int hslot = ucount % NSLOT;
            const float v = reduce_unit(acc, lane);
#pragma unroll
            for (int p = 0; p < TP; ++p)
#pragma unroll
                for (int c = 0; c < 4; ++c) acc[p][c] = 0.f;
            // the hand-over slot is free once the control wave has taken the unit that used it last; its count only
            // grows, so the LDS read is skipped while the last value seen says enough
            if (c_consumed < ucount - NSLOT + 1) {
                Patience pat(8 * budget);
                while ((c_consumed = uni(lds_ld(&sh.consumed))) < ucount - NSLOT + 1) {
                    __builtin_amdgcn_s_sleep(1);
                    if (uni(lds_ld(&sh.abort)) || pat.spent()) { alive = false; break; }
                }
                if (!alive) break;
            }
            {
                // (index recomputed here: as a loop invariant it was kept in a register that the allocator spilled, and its
                // reload waits for every load in flight)
                const int t2 = local_tid(), l2 = t2 & 63;
                if ((l2 & 15) < 3) sh.red[hslot][t2 >> 6][3 * (l2 >> 4) + (l2 & 15)] = v;
            }
            GPTRS_LDS_RELEASE();
            if (lane == 0) __hip_atomic_fetch_add(&sh.red_cnt[hslot], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            ++ucount;
            c_sidx += TP * c_G;
            if (!from_park && r_more) request();
        }
      }   // units
    }
}

template <int FMT, int RING_D>
__global__ __launch_bounds__(NT, 1) void chain_kernel(const ChainPhase* __restrict__ phases, int nphases, unsigned* bar, int* abort_flag,
                                                        int xs_bytes, unsigned long long budget, int stall_phase) {
    extern __shared__ __align__(16) unsigned char smem[];
    Shared& sh = *reinterpret_cast<Shared*>(smem);
    unsigned* xs = reinterpret_cast<unsigned*>(smem + sizeof(Shared));
    unsigned char* ring = smem + sizeof(Shared) + xs_bytes;
    PhaseTable table = (PhaseTable)phases;
    {
        if (threadIdx.x < NSLOT) sh.red_cnt[threadIdx.x] = 0;
        if (threadIdx.x == 0) { sh.go = -1; sh.consumed = 0; sh.abort = 0; }
        __syncthreads();
    }
    const int wave = threadIdx.x >> 6;
    if (wave < NWS) {
        compute_waves<FMT, RING_D>(sh, xs, table, nphases, ring, budget);
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): no load may land in LDS after the workgroup has gone
    } else {
        control_wave<FMT>(sh, xs, phases, nphases, bar, abort_flag, budget, stall_phase);
    }
}

// ---------------------------------------------------------------------------- weight layout
// Wc[tile][j][c][h] = W[2j + h][column(tile, c)], zero outside [K) x [N).  Single: column = 4*tile + c.
// Dual (SwiGLU pair): columns interleaved, c = 0,2 -> gate column 2*tile + c/2, c = 1,3 -> the same
// column of up, so one tile finishes two outputs.
__global__ void chain_pack_kernel(const bf16_t* __restrict__ w, const bf16_t* __restrict__ w2, uint32_t* __restrict__ out,
                                  int64_t K, int64_t N, int64_t Kw, int64_t ntiles) {
    const int64_t total = ntiles * Kw * 4;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
        const int c = (int)(idx & 3);
        const int64_t j = (idx >> 2) % Kw, tile = (idx >> 2) / Kw;
        const bf16_t* src = w;
        int64_t col;
        if (w2) { col = tile * 2 + (c >> 1); if (c & 1) src = w2; }
        else col = tile * 4 + c;
        uint32_t lo = 0, hi = 0;
        if (col < N) {
            if (2 * j < K) lo = src[(2 * j) * N + col];
            if (2 * j + 1 < K) hi = src[(2 * j + 1) * N + col];
        }
        out[idx] = lo | (hi << 16);
    }
}

// Quantised codes: the same tile order with one byte per (column, code row): word j of a tile holds code rows
// 4j .. 4j+3 of its 4 columns.  int8: a code row is one k, bytes stored as q + 128 (flip = 0x80).  int4: a code
// row is a packed byte (k = 2r low nibble, 2r + 1 high nibble), both nibbles stored as q + 8 (flip = 0x88).
// Bytes outside the matrix hold the biased zero.
// f32 weights: word (tile, k) = the 4 columns of the tile at row k
__global__ void chain_pack_f32_kernel(const float* __restrict__ w, float* __restrict__ out, int64_t K, int64_t N, int64_t Kw, int64_t ntiles) {
    const int64_t total = ntiles * Kw * 4;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
        const int c = (int)(idx & 3);
        const int64_t j = (idx >> 2) % Kw, tile = (idx >> 2) / Kw;
        const int64_t col = tile * 4 + c;
        out[idx] = (col < N && j < K) ? w[j * N + col] : 0.f;
    }
}

__global__ void chain_pack_codes_kernel(const uint8_t* __restrict__ w, const uint8_t* __restrict__ w2, uint32_t* __restrict__ out,
                                        int64_t rows, int64_t N, int64_t Kw, int64_t ntiles, uint32_t flip) {
    const int64_t total = ntiles * Kw * 4;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
        const int c = (int)(idx & 3);
        const int64_t j = (idx >> 2) % Kw, tile = (idx >> 2) / Kw;
        const uint8_t* src = w;
        int64_t col;
        if (w2) { col = tile * 2 + (c >> 1); if (c & 1) src = w2; }
        else col = tile * 4 + c;
        uint32_t v = 0;
        for (int h = 0; h < 4; ++h) {
            const int64_t r = 4 * j + h;
            const uint32_t b = (col < N && r < rows) ? ((uint32_t)src[r * N + col] ^ flip) : flip;
            v |= b << (8 * h);
        }
        out[idx] = v;
    }
}
// int4 group scales in tile order: sc[tile][g][c] (bf16) for g < Kw / 16, zero outside the matrix
__global__ void chain_pack_scales_kernel(const bf16_t* __restrict__ sc, const bf16_t* __restrict__ sc2, bf16_t* __restrict__ out,
                                         int64_t groups, int64_t N, int64_t G, int64_t ntiles) {
    const int64_t total = ntiles * G * 4;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
        const int c = (int)(idx & 3);
        const int64_t g = (idx >> 2) % G, tile = (idx >> 2) / G;
        const bf16_t* src = sc;
        int64_t col;
        if (sc2) { col = tile * 2 + (c >> 1); if (c & 1) src = sc2; }
        else col = tile * 4 + c;
        out[idx] = (col < N && g < groups) ? src[g * N + col] : (bf16_t)0;
    }
}

static int g_grid = 0;
static int g_occupancy_ok[8] = {-1, -1, -1, -1, -1, -1, -1, -1};   // per kernel: does a workgroup fit a CU with the LDS it asks for

}  // namespace

int chain_grid() {
    if (g_grid == 0) {
        int dev = 0;
        hipDeviceProp_t prop{};
        if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return 0;
        int g = prop.multiProcessorCount / NC * NC;
        g_grid = g > 0 ? g : -1;
    }
    return g_grid > 0 ? g_grid : 0;
}

static inline int64_t cdiv64(int64_t a, int64_t b) { return (a + b - 1) / b; }
static inline int chain_kpw(int wfmt) { return wfmt == kChainW32 ? 1 : (wfmt == kChainW16 ? 2 : (wfmt == kChainW8 ? 4 : 8)); }   // k per column of a word
// bytes of staged activations per weight word: kpw bf16 values, or one f32
static inline int chain_xbytes(int wfmt) { return wfmt == kChainW32 ? 4 : chain_kpw(wfmt) * 2; }
static inline int64_t chain_kw(int64_t k, int wfmt) { return cdiv64(cdiv64(k, chain_kpw(wfmt)), NS) * NS; }

bool chain_supported(int dtype, int64_t m, int64_t k, int64_t n, bool dual, bool norm, int wfmt, bool x_f32, bool plain) {
    if (m != 1 || k < 4 || n < 4) return false;
    // a width that is not a multiple of 4 (GPT-2's head: 50257): the last tile's missing columns are zero in the copy and are not
    // stored; only for an unquantised layer without bias and residual (staged values and scales come in pairs)
    const bool ragged_ok = plain && !dual && (wfmt == kChainW16 || wfmt == kChainW32);
    if (wfmt < kChainW16 || wfmt > kChainW32) return false;
    if (wfmt == kChainW32) {   // f32 weights, activations and output; no SwiGLU pair
        if (dtype != 0 || dual || k % 4 != 0 || (n % 4 != 0 && !ragged_ok) || k > 4 * (MAXI / 2) * NT) return false;
        return chain_kw(k, wfmt) * chain_xbytes(wfmt) / 4 <= kChainMaxXsWords;
    }
    if (dtype != 2) return false;
    if (x_f32 && (!norm || k > 4 * (MAXI / 2) * NT)) return false;
    if (k % 4 != 0 || (n % (dual ? 2 : 4) != 0 && !ragged_ok)) return false;
    if (wfmt == kChainW4 && k % 128 != 0) return false;
    if (norm && k > 4 * MAXI * NT) return false;
    if (chain_kw(k, wfmt) * chain_xbytes(wfmt) / 4 > kChainMaxXsWords) return false;
    return true;
}

size_t chain_weight_bytes(int64_t k, int64_t n, bool dual, int wfmt) {
    const int64_t ncols = dual ? 2 * n : n;
    return (size_t)(cdiv64(ncols, 4) * chain_kw(k, wfmt) * 16);
}

void chain_pack_weights(hipStream_t s, const void* w, const void* w2, void* out, int64_t k, int64_t n, int wfmt) {
    const int64_t ncols = w2 ? 2 * n : n, ntiles = cdiv64(ncols, 4), kw = chain_kw(k, wfmt);
    const int64_t total = ntiles * kw * 4;
    if (total <= 0) return;
    const unsigned g = (unsigned)std::min<int64_t>(cdiv64(total, 256), 65536);
    if (wfmt == kChainW32)
        chain_pack_f32_kernel<<<g, 256, 0, s>>>((const float*)w, (float*)out, k, n, kw, ntiles);
    else if (wfmt == kChainW16)
        chain_pack_kernel<<<g, 256, 0, s>>>((const bf16_t*)w, (const bf16_t*)w2, (uint32_t*)out, k, n, kw, ntiles);
    else
        chain_pack_codes_kernel<<<g, 256, 0, s>>>((const uint8_t*)w, (const uint8_t*)w2, (uint32_t*)out, wfmt == kChainW8 ? k : k / 2, n, kw,
                                                  ntiles, wfmt == kChainW8 ? 0x80u : 0x88u);
}

size_t chain_scale_bytes(int64_t k, int64_t n, bool dual) {
    return (size_t)(cdiv64(dual ? 2 * n : n, 4) * (chain_kw(k, kChainW4) / 16) * 4 * sizeof(bf16_t));
}

void chain_pack_scales_w4(hipStream_t s, int dtype, const void* sc, const void* sc2, void* out, int64_t k, int64_t n) {
    if (dtype != 2) return;   // the chain only takes bf16 activations and scales
    const int64_t ntiles = cdiv64(sc2 ? 2 * n : n, 4), G = chain_kw(k, kChainW4) / 16;
    const int64_t total = ntiles * G * 4;
    if (total <= 0) return;
    const unsigned g = (unsigned)std::min<int64_t>(cdiv64(total, 256), 65536);
    chain_pack_scales_kernel<<<g, 256, 0, s>>>((const bf16_t*)sc, (const bf16_t*)sc2, (bf16_t*)out, k / 128, n, G, ntiles);
}

bool chain_fill_phase(ChainPhase& p, int64_t k, int64_t n, bool dual, int wfmt) {
    const int grid = chain_grid();
    p.K = (int)k;
    p.N = (int)n;
    p.Kw = (int)chain_kw(k, wfmt);
    p.ntiles = (int)cdiv64(dual ? 2 * n : n, 4);
    p.wpt = p.Kw / NS;
    p.units = (p.ntiles + TP - 1) / TP;
    p.upb = grid > 0 ? (p.units + grid - 1) / grid : p.units;
    p.kind = kChainLinear;
    p.wfmt = wfmt;
    p.lds_bytes = p.Kw * chain_xbytes(wfmt);
    // int4: the workgroup's group scales (8 bytes per tile and group) are staged behind the activations
    const int64_t total = p.lds_bytes + (wfmt == kChainW4 ? (int64_t)p.upb * TP * (p.Kw / 16) * 8 : 0);
    p.lds_total = (int)std::min<int64_t>(total, INT32_MAX);
    if (dual) p.flags |= kChainDual;
    return (int64_t)p.upb * TP * (dual ? 2 : 4) <= EPI_MAX && total <= (int64_t)kChainMaxXsWords * 4;
}

bool chain_attn_supported(int dtype, int64_t t, int64_t n_q, int64_t n_kv, int64_t head_dim, int64_t rot_half) {
    static const bool enabled = [] { const char* e = getenv("GPTRS_HIP_CHAIN_ATTN"); return !(e && e[0] == '0'); }();
    if (!enabled) return false;   // GPTRS_HIP_CHAIN_ATTN=0: decode attention keeps its stand-alone kernels
    if ((dtype != 2 && dtype != 0) || t != 1 || n_kv <= 0 || n_q % n_kv != 0) return false;
    if (dtype == 0 && rot_half != 0) return false;   // f32 rows: no RoPE inside the phase
    const int64_t g = n_q / n_kv;
    if (g != 1 && g != 2 && g != 4 && g != 8) return false;
    if (head_dim != 64 && head_dim != 128 && head_dim != 256) return false;
    if (rot_half != 0 && (rot_half % 8 != 0 || 2 * rot_half > head_dim)) return false;
    return chain_grid() > 0;
}
static int chain_attn_nch(int64_t n_kv) {
    const int64_t n = chain_grid() / n_kv;
    return (int)(n < 1 ? 1 : (n > 64 ? 64 : n));
}
size_t chain_attn_part_bytes(int64_t n_q, int64_t n_kv, int64_t head_dim) {
    return (size_t)n_q * (size_t)chain_attn_nch(n_kv) * (size_t)(head_dim + 2) * sizeof(float);
}
int chain_attn_phases(int64_t capacity) { return capacity <= 128 ? 1 : 2; }
void chain_fill_attn(ChainPhase& partial, ChainPhase& combine, int64_t n_q, int64_t n_kv, int64_t head_dim, int64_t capacity,
                     int64_t rot_half, float scale) {
    const bool single = chain_attn_phases(capacity) == 1;
    const int nch = single ? 1 : chain_attn_nch(n_kv);
    if (single) partial.flags |= kChainAttnFinal;
    for (ChainPhase* p : {&partial, &combine}) {
        p->n_q = (int)n_q; p->n_kv = (int)n_kv; p->head_dim = (int)head_dim; p->capacity = (int)capacity;
        p->rot_half = (int)rot_half; p->nch = nch; p->scale = scale;
    }
    partial.kind = kChainAttnPartial;
    partial.units = (int)n_kv * nch;
    partial.lds_bytes = partial.lds_total = (int)((2 * NWS + NWS * head_dim) * sizeof(float));
    combine.kind = kChainAttnCombine;
    combine.units = (int)n_q;
    combine.lds_bytes = combine.lds_total = (int)(NW * 64 * sizeof(float4));
}

bool chain_launch(hipStream_t s, const ChainPhase* dev_table, int nphases, int lds_bytes, unsigned* bar, int* abort_flag, int wfmt,
                  int stall_phase) {
    const int grid = chain_grid();
    if (grid <= 0 || nphases <= 0 || nphases > kChainMaxPhases || lds_bytes > kChainMaxXsWords * 4) return false;
    if (wfmt < kChainW16 || wfmt > kChainW32) return false;
    const int xs_bytes = (lds_bytes + 1023) / 1024 * 1024;
    static const int max_depth = [] { const char* e = getenv("GPTRS_HIP_CHAIN_RING"); return e ? std::max(RING_MIN, std::min(RING_MAX, atoi(e))) : RING_MAX; }();
    const int depth = sizeof(Shared) + (size_t)xs_bytes + (size_t)max_depth * SLOT_BYTES <= (size_t)LDS_BYTES ? max_depth : RING_MIN;
    const size_t smem = sizeof(Shared) + (size_t)xs_bytes + (size_t)depth * SLOT_BYTES;
    if (smem > (size_t)LDS_BYTES) return false;
    static_assert(RING_MAX == RING_MIN + 1, "two kernels per weight format");
    const int variant = wfmt * 2 + (depth - RING_MIN);
    typedef void (*Kernel)(const ChainPhase*, int, unsigned*, int*, int, unsigned long long, int);
    static const Kernel kernels[8] = {chain_kernel<kChainW16, RING_MIN>, chain_kernel<kChainW16, RING_MAX>, chain_kernel<kChainW8, RING_MIN>,
                                      chain_kernel<kChainW8, RING_MAX>,  chain_kernel<kChainW4, RING_MIN>,  chain_kernel<kChainW4, RING_MAX>,
                                      chain_kernel<kChainW32, RING_MIN>, chain_kernel<kChainW32, RING_MAX>};
    static_assert(kChainW16 == 0 && kChainW8 == 1 && kChainW4 == 2 && kChainW32 == 3, "index of a kernel");
    const Kernel fn = kernels[variant];
    if (g_occupancy_ok[variant] < 0) {
        // The grid barrier needs every workgroup resident at once: one workgroup per CU, grid <= CUs (chain_grid), and the
        // kernel with the LDS it asks for must fit a CU.  Checked once per kernel.
        int per_cu = 0;
        const bool ok = hipFuncSetAttribute((const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES) == hipSuccess &&
                        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void*)fn, NT, smem) == hipSuccess && per_cu >= 1;
        g_occupancy_ok[variant] = ok ? 1 : 0;
    }
    if (!g_occupancy_ok[variant]) return false;
    // wall-clock budget of a grid-barrier wait, in ticks of the 100 MHz counter (GPTRS_HIP_CHAIN_WAIT_MS, default 50 ms;
    // a stalled test launch gets 2 ms)
    static const unsigned long long budget = [] {
        const char* e = getenv("GPTRS_HIP_CHAIN_WAIT_MS");
        const long ms = e ? atol(e) : 50;
        return (unsigned long long)std::max<long>(1, std::min<long>(ms, 10000)) * 100000ull;
    }();
    const unsigned long long ticks = stall_phase >= 0 ? 200000ull : budget;
    fn<<<grid, NT, smem, s>>>(dev_table, nphases, bar, abort_flag, xs_bytes, ticks, stall_phase);
    return true;
}

}  // namespace k
}  // namespace gptrs
