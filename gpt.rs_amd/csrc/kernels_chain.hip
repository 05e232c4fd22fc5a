// Decode linear layers as ONE persistent launch per run of consecutive linears ("chain").
//
// A decode step of a transformer block is a dependent sequence of GEMVs (out-proj -> gate/up ->
// down -> next block's qkv ...), each streaming tens of MB of weights once.  Launched one by one,
// every GEMV pays a launch gap, a cold start and a tail; here the whole run executes inside one
// kernel of one workgroup per CU, phases separated by a grid-wide barrier:
//
//   * 8 streaming waves per workgroup only load weight words and issue v_dot2 (bf16 pairs): a
//     workgroup owns groups of TP tiles of 4 output columns for the whole of K, lane t reading word
//     t, t+512, ... of each tile stream (Wc[tile][k/2][4 cols][2 k], 16-byte words).  The next
//     j-step (TP words) is always in flight while the current one is consumed, across unit AND phase
//     boundaries: weights do not depend on activations, so the first words of the next layer are
//     already in registers when its input becomes ready.
//   * 1 control wave per workgroup sums the 8 waves' partial sums of a unit out of LDS, applies the
//     epilogue (SwiGLU pair, bias, GELU, residual), stores through to memory, and runs the grid
//     barrier (16 striped arrival counters, one poll instruction).
//   * Activations cross workgroups through agent-scope (sc1) loads and stores only, so no
//     L2 write-back / invalidate is needed between phases; a phase's input vector is staged into
//     LDS by all 9 waves together right after the barrier (RMSNorm statistics included).
//
// Every wait is bounded: a barrier that does not complete raises the abort flag, every wave
// leaves the kernel, and the host reports an execution error.
#include <algorithm>

#include "kernels.hpp"
#include "device_utils.hpp"

namespace gptrs {
namespace k {

namespace {

constexpr int NS = 512;          // streaming threads
constexpr int NT = NS + 64;      // + control wave
constexpr int NWS = NS / 64;
constexpr int TP = 3;            // tiles (of 4 columns) per unit
constexpr int NSLOT = 4;         // unit hand-off slots between streaming waves and control wave
constexpr int NC = kChainCounters;
constexpr int EPI_MAX = 2048;    // bias/residual values staged per workgroup and phase
constexpr int MAXI = 8;          // 8-byte items per thread in the norm staging: K <= 4*MAXI*NT

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }
template <typename T> __device__ __forceinline__ T* uni_ptr(T* p) {
    const unsigned long long v = (unsigned long long)p;
    const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)v);
    const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(v >> 32));
    return (T*)(((unsigned long long)hi << 32) | lo);
}
// agent-scope accesses: coherent across the XCDs' L2s without cache maintenance
__device__ __forceinline__ unsigned long long cload8(const void* p) {
    return __hip_atomic_load((const unsigned long long*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned cload4(const void* p) {
    return __hip_atomic_load((const unsigned*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void cstore8(void* p, unsigned long long v) {
    __hip_atomic_store((unsigned long long*)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void cstore4(void* p, unsigned v) {
    __hip_atomic_store((unsigned*)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float rbf(float v) { return bf16_to_f32(f32_to_bf16(v)); }
__device__ __forceinline__ int lds_ld(const int* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP); }
__device__ __forceinline__ void lds_st(int* p, int v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP); }
#define GPTRS_LDS_RELEASE() __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local")
#define GPTRS_LDS_ACQUIRE() __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local")
// workgroup barrier that waits for LDS traffic only: outstanding weight loads stay in flight
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
}

struct Shared {
    float red[NSLOT][NWS][16];
    float epi_bias[EPI_MAX];
    float epi_res[EPI_MAX];
    float ssq[16];
    int red_cnt[NSLOT];
    int go, consumed, abort, pad;
    ChainPhase ph[kChainMaxPhases];
};

// ---------------------------------------------------------------------------- staging (all waves)
// xs[j] = (x[2j], x[2j+1]) as a bf16 pair, zero beyond K; with norm: the value the stand-alone
// RMSNorm kernel stores, ((x * inv_rms) -> bf16) * gamma -> bf16 (normalization.rs:183-217).
__device__ void stage_block(const ChainPhase& P, unsigned* xs, float* ssq) {
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int K = uni(P.K), Kw = uni(P.Kw);
    const int n = K / 4;        // 8-byte items holding data (K % 4 == 0)
    const int npad = Kw / 2;    // items to write
    const char* x = (const char*)uni_ptr(P.x);
    if (uni(P.flags) & kChainNorm) {
        const uint2* g = (const uint2*)uni_ptr(P.gamma);
        unsigned long long v[MAXI];
        uint2 gg[MAXI];
#pragma unroll
        for (int u = 0; u < MAXI; ++u) {
            const int i = u * NT + t;
            v[u] = i < n ? cload8(x + 8 * (size_t)i) : 0ull;
            gg[u] = i < n ? g[i] : make_uint2(0u, 0u);
        }
        float q = 0.f;
#pragma unroll
        for (int u = 0; u < MAXI; ++u) {
            const unsigned lo = (unsigned)v[u], hi = (unsigned)(v[u] >> 32);
            const float a = bf16lo(lo), b = bf16hi(lo), c = bf16lo(hi), d = bf16hi(hi);
            q += a * a; q += b * b; q += c * c; q += d * d;
        }
        const float ws = wave_sum(q);
        if (lane == 0) ssq[wave] = ws;
        lds_barrier();
        float tot = 0.f;
#pragma unroll
        for (int w = 0; w < NT / 64; ++w) tot += ssq[w];
        const float inv = 1.0f / sqrtf(tot * P.inv_n + P.eps);
#pragma unroll
        for (int u = 0; u < MAXI; ++u) {
            const int i = u * NT + t;
            if (i < npad) {
                const unsigned lo = (unsigned)v[u], hi = (unsigned)(v[u] >> 32);
                const unsigned o0 = pack_bf16x2(rbf(bf16lo(lo) * inv) * bf16lo(gg[u].x), rbf(bf16hi(lo) * inv) * bf16hi(gg[u].x));
                const unsigned o1 = pack_bf16x2(rbf(bf16lo(hi) * inv) * bf16lo(gg[u].y), rbf(bf16hi(hi) * inv) * bf16hi(gg[u].y));
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
    lds_barrier();
}

// ---------------------------------------------------------------------------- control wave
__device__ __forceinline__ float finish(float v, int flags, float bias, float res) {
    if (flags & kChainBias) v += bias;                                           // tensor_ops.rs:42-56
    if (flags & kChainGelu) v = (v * 0.5f) * (erff(v / 1.41421354f) + 1.0f);     // activation.rs:96-113
    if (flags & kChainResidual) v += res;
    return v;
}

__device__ void control_wave(Shared& sh, unsigned* xs, int nphases, unsigned* bar, int* abort_flag) {
    const int lane = threadIdx.x & 63;
    const int blk = blockIdx.x, per = gridDim.x / NC;
    const unsigned epoch = bar[NC * 64];   // written by the previous launch, stable during this one
    int ucount = 0;
    for (int ph = 0; ph < nphases; ++ph) {
        const ChainPhase& P = sh.ph[ph];
        const int upb = uni(P.upb), units = uni(P.units);
        const int u0 = blk * upb, u1 = min(u0 + upb, units);
        if (ph > 0) {
            const unsigned target = epoch + (unsigned)ph * per;
            unsigned spins = 0;
            bool ok = true;
            for (;;) {
                const unsigned v = lane < NC ? __hip_atomic_load(bar + lane * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : target;
                if (__builtin_amdgcn_ballot_w64((int)(v - target) < 0) == 0) break;
                __builtin_amdgcn_s_sleep(1);
                if ((++spins & 63u) == 0) {
                    if (__hip_atomic_load(abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) || spins > (1u << 19)) { ok = false; break; }
                }
            }
            if (!ok) {
                __hip_atomic_store(abort_flag, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                lds_st(&sh.abort, 1);
                return;
            }
        }
        if (u0 < u1) {
            const int flags = uni(P.flags), ntiles = uni(P.ntiles), N = uni(P.N);
            const bool dual = flags & kChainDual;
            const int cpt = dual ? 2 : 4;              // output columns per tile
            const int col0 = u0 * TP * cpt;
            const int ncols = min((u1 - u0) * TP * cpt, EPI_MAX);
            // bias / residual of this workgroup's columns: requested before the staging loads so
            // their latency hides behind the staging
            const unsigned* bias = (const unsigned*)uni_ptr(P.bias);
            const char* resid = (const char*)uni_ptr(P.residual);
            if (lane == 0) lds_st(&sh.go, ph);
            if (bias || resid) {
                for (int i = lane * 2; i < ncols; i += 128) {
                    const int col = col0 + i;
                    const unsigned bw = (bias && col < N) ? bias[col >> 1] : 0u;
                    const unsigned rw = (resid && col < N) ? cload4(resid + 2 * (size_t)col) : 0u;
                    *reinterpret_cast<float2*>(&sh.epi_bias[i]) = make_float2(bf16lo(bw), bf16hi(bw));
                    *reinterpret_cast<float2*>(&sh.epi_res[i]) = make_float2(bf16lo(rw), bf16hi(rw));
                }
            }
            stage_block(P, xs, sh.ssq);
            char* out = (char*)uni_ptr(P.y);
            for (int u = u0; u < u1; ++u, ++ucount) {
                const int slot = ucount % NSLOT;
                unsigned spins = 0;
                while (lds_ld(&sh.red_cnt[slot]) < NWS) {
                    __builtin_amdgcn_s_sleep(1);
                    if (++spins > (1u << 24)) {
                        lds_st(&sh.abort, 1);
                        __hip_atomic_store(abort_flag, 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
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
                    if (dual) {   // columns interleaved (gate, up, gate, up): activation.rs:141-162
                        const float a0 = finish((s[0] / (1.0f + expf(s[0] * -1.0f))) * s[1], flags, sh.epi_bias[e], sh.epi_res[e]);
                        const float a1 = finish((s[2] / (1.0f + expf(s[2] * -1.0f))) * s[3], flags, sh.epi_bias[e + 1], sh.epi_res[e + 1]);
                        cstore4(out + 2 * (size_t)(tile * 2), pack_bf16x2(a0, a1));
                    } else {
                        float o[4];
#pragma unroll
                        for (int c = 0; c < 4; ++c) o[c] = finish(s[c], flags, sh.epi_bias[e + c], sh.epi_res[e + c]);
                        cstore8(out + 2 * (size_t)(tile * 4),
                                (unsigned long long)pack_bf16x2(o[0], o[1]) | ((unsigned long long)pack_bf16x2(o[2], o[3]) << 32));
                    }
                }
            }
        }
        // this workgroup's outputs have left the CU before it arrives at the barrier
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        asm volatile("" ::: "memory");
        if (lane == 0) __hip_atomic_fetch_add(bar + (blk % NC) * 64, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    // every launch advances each counter by nphases * per: the next launch starts from there
    if (blk == 0 && lane == 0) bar[NC * 64] = epoch + (unsigned)nphases * per;
}

// ---------------------------------------------------------------------------- streaming waves
__device__ void stream_waves(Shared& sh, const unsigned* xs, int nphases) {
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int blk = blockIdx.x;

    // load iterator: the next j-step (TP words per lane) to fetch
    int l_phase = -1, l_unit = 0, l_unit_end = 0, l_j = 0, l_wpt = 1, l_ntiles = 1;
    long l_Kw = 0;
    const uint4* l_w = nullptr;
    bool l_active = true;
    const uint4* l_base[TP];
#pragma unroll
    for (int p = 0; p < TP; ++p) l_base[p] = nullptr;
    auto l_setbase = [&]() {
#pragma unroll
        for (int p = 0; p < TP; ++p) {
            const int tile = min(l_unit * TP + p, l_ntiles - 1);   // a group's last tiles may not exist: re-read, never stored
            l_base[p] = l_w + (long)tile * l_Kw + t;
        }
        l_j = 0;
    };
    auto l_seek = [&]() {
        while (l_active && l_unit >= l_unit_end) {
            ++l_phase;
            if (l_phase >= nphases) { l_active = false; break; }
            const ChainPhase& ph = sh.ph[l_phase];
            const int upb = uni(ph.upb), units = uni(ph.units);
            l_unit = blk * upb;
            l_unit_end = min(l_unit + upb, units);
            if (l_unit < l_unit_end) {
                l_wpt = uni(ph.wpt); l_ntiles = uni(ph.ntiles); l_Kw = uni(ph.Kw);
                l_w = (const uint4*)uni_ptr(ph.w);
            }
        }
        if (l_active) l_setbase();
    };
    auto l_fetch = [&](uint4 (&dst)[TP]) {   // requires l_active
#pragma unroll
        for (int p = 0; p < TP; ++p) dst[p] = l_base[p][(long)l_j * NS];
        if (++l_j == l_wpt) {
            ++l_unit;
            if (l_unit >= l_unit_end) l_seek(); else l_setbase();
        }
    };

    // compute iterator
    int c_phase = -1, c_unit = 0, c_unit_end = 0, c_j = 0, c_wpt = 1, ucount = 0;
    auto c_seek = [&]() -> bool {
        while (c_unit >= c_unit_end) {
            ++c_phase;
            if (c_phase >= nphases) return false;
            const ChainPhase& ph = sh.ph[c_phase];
            const int upb = uni(ph.upb), units = uni(ph.units);
            c_unit = blk * upb;
            c_unit_end = min(c_unit + upb, units);
            if (c_unit < c_unit_end) {
                c_wpt = uni(ph.wpt);
                unsigned spins = 0;
                while (uni(lds_ld(&sh.go)) < c_phase) {
                    __builtin_amdgcn_s_sleep(1);
                    if (uni(lds_ld(&sh.abort)) || ++spins > (1u << 24)) return false;
                }
                stage_block(sh.ph[c_phase], const_cast<unsigned*>(xs), sh.ssq);
            }
        }
        c_j = 0;
        return true;
    };

    uint4 cur[TP], nxt[TP];
    bool have_nxt = false;
    l_seek();
    if (l_active) { l_fetch(nxt); have_nxt = true; }
    float acc[TP][4];
#pragma unroll
    for (int p = 0; p < TP; ++p)
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[p][c] = 0.f;

    bool alive = c_seek();
    while (alive && have_nxt) {
#pragma unroll
        for (int p = 0; p < TP; ++p) cur[p] = nxt[p];
        if (l_active) l_fetch(nxt); else have_nxt = false;
        const bf16x2 xv = __builtin_bit_cast(bf16x2, xs[c_j * NS + t]);
#pragma unroll
        for (int p = 0; p < TP; ++p) {
            const uint4 q = cur[p];
            acc[p][0] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, q.x), xv, acc[p][0], false);
            acc[p][1] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, q.y), xv, acc[p][1], false);
            acc[p][2] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, q.z), xv, acc[p][2], false);
            acc[p][3] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, q.w), xv, acc[p][3], false);
        }
        if (++c_j == c_wpt) {
            const int slot = ucount % NSLOT;
            float v = 0.f;
#pragma unroll
            for (int p = 0; p < TP; ++p)
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const float a = wave_sum(acc[p][c]);
                    if (lane == p * 4 + c) v = a;
                    acc[p][c] = 0.f;
                }
            unsigned spins = 0;
            while (uni(lds_ld(&sh.consumed)) < ucount - NSLOT + 1) {
                __builtin_amdgcn_s_sleep(1);
                if (uni(lds_ld(&sh.abort)) || ++spins > (1u << 24)) return;
            }
            if (lane < TP * 4) sh.red[slot][wave][lane] = v;
            GPTRS_LDS_RELEASE();
            if (lane == 0) __hip_atomic_fetch_add(&sh.red_cnt[slot], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            ++ucount;
            ++c_unit;
            if (c_unit >= c_unit_end) alive = c_seek(); else c_j = 0;
        }
    }
}

__global__ __launch_bounds__(NT, 1) void chain_kernel(const ChainPhase* __restrict__ phases, int nphases, unsigned* bar, int* abort_flag) {
    extern __shared__ __align__(16) unsigned char smem[];
    Shared& sh = *reinterpret_cast<Shared*>(smem);
    unsigned* xs = reinterpret_cast<unsigned*>(smem + sizeof(Shared));
    {
        const int* src = (const int*)phases;
        int* dst = (int*)sh.ph;
        const int nw = nphases * (int)(sizeof(ChainPhase) / 4);
        for (int i = threadIdx.x; i < nw; i += NT) dst[i] = src[i];
        if (threadIdx.x < NSLOT) sh.red_cnt[threadIdx.x] = 0;
        if (threadIdx.x == 0) { sh.go = -1; sh.consumed = 0; sh.abort = 0; }
        __syncthreads();
    }
    if (threadIdx.x >= NS) control_wave(sh, xs, nphases, bar, abort_flag);
    else stream_waves(sh, xs, nphases);
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

static int g_grid = 0;
static size_t g_smem_set = 0;

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

bool chain_supported(int dtype, int64_t m, int64_t k, int64_t n, bool dual, bool norm) {
    if (dtype != 2 || m != 1 || k < 4 || n < 4) return false;
    if (k % 4 != 0 || n % (dual ? 2 : 4) != 0) return false;
    if (norm && k > 4 * MAXI * NT) return false;
    if (k > 2 * kChainMaxXsWords) return false;
    return true;
}

static inline int64_t cdiv64(int64_t a, int64_t b) { return (a + b - 1) / b; }
static inline int64_t chain_kw(int64_t k) { return cdiv64(cdiv64(k, 2), NS) * NS; }

size_t chain_weight_bytes(int64_t k, int64_t n, bool dual) {
    const int64_t ncols = dual ? 2 * n : n;
    return (size_t)(cdiv64(ncols, 4) * chain_kw(k) * 16);
}

void chain_pack_weights(hipStream_t s, const void* w, const void* w2, void* out, int64_t k, int64_t n) {
    const int64_t ncols = w2 ? 2 * n : n, ntiles = cdiv64(ncols, 4), kw = chain_kw(k);
    const int64_t total = ntiles * kw * 4;
    if (total <= 0) return;
    const unsigned g = (unsigned)std::min<int64_t>(cdiv64(total, 256), 65536);
    chain_pack_kernel<<<g, 256, 0, s>>>((const bf16_t*)w, (const bf16_t*)w2, (uint32_t*)out, k, n, kw, ntiles);
}

bool chain_fill_phase(ChainPhase& p, int64_t k, int64_t n, bool dual) {
    const int grid = chain_grid();
    p.K = (int)k;
    p.N = (int)n;
    p.Kw = (int)chain_kw(k);
    p.ntiles = (int)cdiv64(dual ? 2 * n : n, 4);
    p.wpt = p.Kw / NS;
    p.units = (p.ntiles + TP - 1) / TP;
    p.upb = grid > 0 ? (p.units + grid - 1) / grid : p.units;
    if (dual) p.flags |= kChainDual;
    return (int64_t)p.upb * TP * (dual ? 2 : 4) <= EPI_MAX && p.Kw <= kChainMaxXsWords;
}

bool chain_launch(hipStream_t s, const ChainPhase* dev_table, int nphases, int max_kw, unsigned* bar, int* abort_flag) {
    const int grid = chain_grid();
    if (grid <= 0 || nphases <= 0 || nphases > kChainMaxPhases || max_kw > kChainMaxXsWords) return false;
    const size_t smem = sizeof(Shared) + (size_t)max_kw * 4;
    if (smem > g_smem_set) {
        const size_t want = sizeof(Shared) + (size_t)kChainMaxXsWords * 4;
        if (hipFuncSetAttribute((const void*)chain_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)want) != hipSuccess) return false;
        g_smem_set = want;
    }
    chain_kernel<<<grid, NT, smem, s>>>(dev_table, nphases, bar, abort_flag);
    return true;
}

}  // namespace k
}  // namespace gptrs
