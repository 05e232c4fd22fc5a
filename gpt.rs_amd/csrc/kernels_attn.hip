// Causal attention kernels for the two sequences the reference emits:
//   * attention_decode_cache (crates/gpt-rs/src/ops/functional/attention.rs:657-779), T = 1
//   * attention without cache (attention.rs:443-522), prefill
// Both compute softmax((q.k) * scale + mask) . v with the additive -1e9 mask replaced by its
// exact f32 effect: masked positions contribute exactly 0 (exp underflows), so only positions
// <= the query position are visited.  GQA: query head h reads kv head h / group.
#include <cstdlib>

#include "kernels.hpp"
#include "device_utils.hpp"

namespace gptrs {
namespace k {

static inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

template <typename T> __device__ __forceinline__ float ldf(const T* p, int64_t i);
template <> __device__ __forceinline__ float ldf<float>(const float* p, int64_t i) { return p[i]; }
template <> __device__ __forceinline__ float ldf<bf16_t>(const bf16_t* p, int64_t i) { return bf16_to_f32(p[i]); }
template <typename T> __device__ __forceinline__ void stf(T* p, int64_t i, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, int64_t i, float v) { p[i] = v; }
template <> __device__ __forceinline__ void stf<bf16_t>(bf16_t* p, int64_t i, float v) { p[i] = f32_to_bf16(v); }

template <typename T> struct Vec16;
template <> struct Vec16<float> {
    static constexpr int N = 4;
    static __device__ __forceinline__ void load(const float* p, float (&o)[4]) {
        const float4 v = *reinterpret_cast<const float4*>(p);
        o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
    }
};
template <> struct Vec16<bf16_t> {
    static constexpr int N = 8;
    static __device__ __forceinline__ void load(const bf16_t* p, float (&o)[8]) {
        const uint4 v = *reinterpret_cast<const uint4*>(p);
        o[0] = bf16lo(v.x); o[1] = bf16hi(v.x); o[2] = bf16lo(v.y); o[3] = bf16hi(v.y);
        o[4] = bf16lo(v.z); o[5] = bf16hi(v.z); o[6] = bf16lo(v.w); o[7] = bf16hi(v.w);
    }
};

constexpr int kMaxDecodeSplits = 512;

typedef __bf16 bf16x8_v __attribute__((ext_vector_type(8)));
typedef float f32x16_v __attribute__((ext_vector_type(16)));

__device__ __forceinline__ int64_t clamp_i64(int64_t v, int64_t lo, int64_t hi) { return v < lo ? lo : (v > hi ? hi : v); }

// Rotate-half RoPE (ops/functional/rotary.rs:430-536) applied while loading VEC consecutive dims
// [c0, c0+VEC) of one head: dims below `half` pair with dim+half, the next `half` dims pair with
// dim-half, dims >= 2*half pass through.  Needs half % VEC == 0 so a chunk never straddles a
// boundary.  The result is rounded to T, the value a stored post-RoPE row would hold.
template <typename T>
__device__ __forceinline__ void load_roped(const T* __restrict__ head, int c0, int half, const T* __restrict__ cs,
                                           const T* __restrict__ sn, float (&out)[Vec16<T>::N]) {
    constexpr int VEC = Vec16<T>::N;
    float own[VEC];
    Vec16<T>::load(head + c0, own);
    if (c0 >= 2 * half) {
#pragma unroll
        for (int v = 0; v < VEC; ++v) out[v] = own[v];
        return;
    }
    const bool first = c0 < half;
    float other[VEC], c[VEC], s[VEC];
    Vec16<T>::load(head + (first ? c0 + half : c0 - half), other);
    const int j0 = first ? c0 : c0 - half;
    Vec16<T>::load(cs + j0, c);
    Vec16<T>::load(sn + j0, s);
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
        // first half: a*cos - b*sin with (a,b) = (own, other); second half: b*cos + a*sin with (b,a) = (own, other)
        const float r = first ? own[v] * c[v] - other[v] * s[v] : own[v] * c[v] + other[v] * s[v];
        T tmp;
        stf(&tmp, 0, r);
        out[v] = ldf(&tmp, 0);
    }
}
template <typename T>
__device__ __forceinline__ T roped_elem(const T* __restrict__ head, int d, int half, const T* __restrict__ cs,
                                        const T* __restrict__ sn) {
    if (d >= 2 * half) return head[d];
    const bool first = d < half;
    const int j = first ? d : d - half;
    const float own = ldf(head, d), other = ldf(head, first ? d + half : d - half);
    const float r = first ? own * ldf(cs, j) - other * ldf(sn, j) : own * ldf(cs, j) + other * ldf(sn, j);
    T tmp;
    stf(&tmp, 0, r);
    return tmp;
}

// ------------------------------------------------------------------------------ decode
// grid (n_kv, nsplit), 256 threads.  A cache row (head_dim elements) is read by LPR lanes with one
// 16-byte load each, so a wave streams 64/LPR positions at a time; every such lane-group keeps
// its own online-softmax state for the G query heads of this kv head.  States are merged by
// shuffles inside the wave, through LDS across the four waves, and across splits by
// attn_decode_combine_kernel.
struct DecodeCaches { void* k[16]; void* v[16]; };   // per-sequence cache pointers of a batched launch (blockIdx.z)

template <typename T, int G>
__global__ __launch_bounds__(256) void attn_decode_kernel(const T* __restrict__ qkv, T* __restrict__ kc,
                                                          T* __restrict__ vc, const int32_t* __restrict__ us,
                                                          const int32_t* __restrict__ qs, T* __restrict__ ctx,
                                                          float* __restrict__ ws, int n_q, int n_kv, int dh,
                                                          int64_t cap, float scale, int64_t chunk, int nsplit,
                                                          const T* __restrict__ cs, const T* __restrict__ sn, int half,
                                                          int batched, DecodeCaches caches) {
    if (batched) {   // sequence blockIdx.z: its row of the stacked projection and of the context, its caches, its records
        const int b = blockIdx.z;
        kc = (T*)caches.k[b];
        vc = (T*)caches.v[b];
        qkv += (int64_t)b * (n_q + 2 * n_kv) * dh;
        ctx += (int64_t)b * n_q * dh;
        ws += (int64_t)b * n_q * nsplit * (dh + 2);
    }
    constexpr int VEC = Vec16<T>::N;
    const int lpr = dh / VEC;          // lanes per cache row (power of two, <= 64)
    const int rpw = 64 / lpr;          // rows per wave-iteration
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane / lpr, li = lane % lpr;
    const int nstream = 4 * rpw, sid = wave * rpw + sub;
    const int kvh = blockIdx.x, split = blockIdx.y;

    const int64_t qpos = clamp_i64(qs[0], 0, cap - 1);   // DynamicSlice clamp (cpu.rs:804-820)
    const int64_t upd = clamp_i64(us[1], 0, cap - 1);    // DynamicUpdateSlice clamp on the position axis
    const T* knew = qkv + (int64_t)n_q * dh + (int64_t)kvh * dh;
    const T* vnew = qkv + (int64_t)(n_q + n_kv) * dh + (int64_t)kvh * dh;

    // append this step's row (exactly one block per kv head owns position `upd`)
    if (upd / chunk == split) {
        for (int d = threadIdx.x; d < dh; d += 256) {
            kc[((int64_t)kvh * cap + upd) * dh + d] = cs ? roped_elem<T>(knew, d, half, cs, sn) : knew[d];
            vc[((int64_t)kvh * cap + upd) * dh + d] = vnew[d];
        }
    }

    const int64_t p0 = (int64_t)split * chunk;
    int64_t p1 = p0 + chunk;
    if (p1 > qpos + 1) p1 = qpos + 1;

    float qf[G][VEC];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const T* qh = qkv + (int64_t)(kvh * G + g) * dh;
        if (cs) load_roped<T>(qh, li * VEC, half, cs, sn, qf[g]);
        else Vec16<T>::load(qh + li * VEC, qf[g]);
    }

    float m[G], l[G], o[G][VEC];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        m[g] = -INFINITY; l[g] = 0.f;
#pragma unroll
        for (int v = 0; v < VEC; ++v) o[g][v] = 0.f;
    }

    // Two positions per lane-group are loaded before either is consumed (the kernel is bound by
    // load latency, not bandwidth); a position past the end re-reads a valid row and is skipped.
    for (int64_t base = p0 + sid; base < p1; base += 2 * nstream) {
        float kf2[2][VEC], vf2[2][VEC];
        bool live[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int64_t p = base + (int64_t)j * nstream;
            live[j] = p < p1;
            const int64_t pc = live[j] ? p : base;
            const bool fresh = pc == upd;
            const T* kr = fresh ? knew : kc + ((int64_t)kvh * cap + pc) * dh;
            const T* vr = fresh ? vnew : vc + ((int64_t)kvh * cap + pc) * dh;
            if (cs && fresh) load_roped<T>(knew, li * VEC, half, cs, sn, kf2[j]);
            else Vec16<T>::load(kr + li * VEC, kf2[j]);
            Vec16<T>::load(vr + li * VEC, vf2[j]);
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
        if (!live[j]) continue;
        const float (&kf)[VEC] = kf2[j];
        const float (&vf)[VEC] = vf2[j];
#pragma unroll
        for (int g = 0; g < G; ++g) {
            float s = 0.f;
#pragma unroll
            for (int v = 0; v < VEC; ++v) s += qf[g][v] * kf[v];
            for (int off = 1; off < lpr; off <<= 1) s += __shfl_xor(s, off, 64);
            s *= scale;
            const float mn = fmaxf(m[g], s);
            const float corr = expf(m[g] - mn);
            const float pe = expf(s - mn);
            l[g] = l[g] * corr + pe;
#pragma unroll
            for (int v = 0; v < VEC; ++v) o[g][v] = o[g][v] * corr + pe * vf[v];
            m[g] = mn;
        }
        }
    }

    // merge the rpw lane-groups of this wave
    for (int off = lpr; off < 64; off <<= 1) {
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const float om = __shfl_xor(m[g], off, 64);
            const float ol = __shfl_xor(l[g], off, 64);
            const float mn = fmaxf(m[g], om);
            const float ca = mn == -INFINITY ? 0.f : expf(m[g] - mn);
            const float cb = mn == -INFINITY ? 0.f : expf(om - mn);
            l[g] = l[g] * ca + ol * cb;
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
                const float ov = __shfl_xor(o[g][v], off, 64);
                o[g][v] = o[g][v] * ca + ov * cb;
            }
            m[g] = mn;
        }
    }

    // merge the four waves through LDS
    __shared__ float sm[4][G], sl[4][G];
    __shared__ float so[4][G][256];
    if (sub == 0) {
#pragma unroll
        for (int g = 0; g < G; ++g) {
            if (li == 0) { sm[wave][g] = m[g]; sl[wave][g] = l[g]; }
#pragma unroll
            for (int v = 0; v < VEC; ++v) so[wave][g][li * VEC + v] = o[g][v];
        }
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < G * dh; idx += 256) {
        const int g = idx / dh, d = idx % dh;
        float mn = fmaxf(fmaxf(sm[0][g], sm[1][g]), fmaxf(sm[2][g], sm[3][g]));
        float L = 0.f, O = 0.f;
        if (mn != -INFINITY) {
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const float c = expf(sm[w][g] - mn);
                L += sl[w][g] * c;
                O += so[w][g][d] * c;
            }
        }
        const int h = kvh * G + g;
        if (nsplit == 1) {
            stf(ctx, (int64_t)h * dh + d, O / L);
        } else {
            float* rec = ws + ((int64_t)h * nsplit + split) * (dh + 2);
            if (d == 0) { rec[0] = mn; rec[1] = L; }
            rec[2 + d] = O;
        }
    }
}

// max / sum of a value over the two half-waves, in every lane: v_permlane32_swap leaves the low half's value in one
// register and the high half's in the other (one VALU instruction instead of a round trip through the LDS crossbar)
__device__ __forceinline__ float half_max(float x) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float half_sum(float x) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
// bf16 decode attention with the scores on the matrix cores.  grid (n_kv, nsplit, batch), 256 threads; wave w of a
// workgroup takes the 32-key tiles w, w+4, ... of the workgroup's chunk.  Per tile
//   S^T[key, q] = K[key, :] . Q[q, :]   v_mfma_f32_32x32x16_bf16, A = cache rows straight from memory (lane = key row),
//                                       B = the group's G query heads in columns 0..G-1 (other columns repeat them)
// so a lane owns ONE query: its 16 scores, the running maximum and sum (log2 domain) are per-lane values and the
// softmax costs a few instructions per key instead of a cross-lane reduction per key and head.  The probabilities go
// through LDS to the layout of the second product, which stays on the vector ALUs in f32: lane-group `sub` (DH/8
// lanes, 16 bytes of a V row each) accumulates O[g, :] over its keys of the tile.  States are merged across
// lane-groups by shuffles, across waves through LDS, across splits by attn_decode_combine_kernel (same records as
// attn_decode_kernel, maxima in natural-log units).
template <int DH, int G>
__global__ __launch_bounds__(256) void attn_decode_mfma_kernel(const bf16_t* __restrict__ qkv, bf16_t* __restrict__ kc,
                                                               bf16_t* __restrict__ vc, const int32_t* __restrict__ us,
                                                               const int32_t* __restrict__ qs, bf16_t* __restrict__ ctx,
                                                               float* __restrict__ ws, int n_q, int n_kv, int64_t cap,
                                                               float scale_log2e, int64_t chunk, int nsplit,
                                                               const bf16_t* __restrict__ cs, const bf16_t* __restrict__ sn,
                                                               int half_rot, int batched, DecodeCaches caches) {
    constexpr int NK = DH / 16;        // k-steps of the score product
    constexpr int LPR = DH / 8;        // lanes per V row
    constexpr int NSUB = 64 / LPR;     // lane-groups per wave
    constexpr int NV = 32 / NSUB;      // keys of a tile per lane-group
    __shared__ __align__(16) float p_lds[2][4][G][32];
    __shared__ float corr_lds[2][4][G];
    __shared__ float sm[4][G], sl[4][G];
    __shared__ float so[4][G][DH];
    __shared__ __align__(16) bf16_t q_lds[G][DH];
    if (batched) {
        const int b = blockIdx.z;
        kc = (bf16_t*)caches.k[b];
        vc = (bf16_t*)caches.v[b];
        qkv += (int64_t)b * (n_q + 2 * n_kv) * DH;
        ctx += (int64_t)b * n_q * DH;
        ws += (int64_t)b * n_q * nsplit * (DH + 2);
    }
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, half = lane >> 5;
    const int sub = lane / LPR, li = lane % LPR;
    const int kvh = blockIdx.x, split = blockIdx.y;
    const int64_t qpos = clamp_i64(qs[0], 0, cap - 1);
    const int64_t upd = clamp_i64(us[1], 0, cap - 1);
    const bf16_t* knew = qkv + (int64_t)n_q * DH + (int64_t)kvh * DH;
    const bf16_t* vnew = qkv + (int64_t)(n_q + n_kv) * DH + (int64_t)kvh * DH;
    bf16_t* kbase = kc + (int64_t)kvh * cap * DH;
    bf16_t* vbase = vc + (int64_t)kvh * cap * DH;

    // append this step's row (one workgroup per kv head owns position `upd`); the rows are read back below, by this
    // workgroup only, after the barrier
    if (upd / chunk == split) {
        for (int d = tid; d < DH; d += 256) {
            kbase[upd * DH + d] = cs ? roped_elem<bf16_t>(knew, d, half_rot, cs, sn) : knew[d];
            vbase[upd * DH + d] = vnew[d];
        }
        __threadfence_block();
    }
    // the group's query heads, rotated once per workgroup (16 bytes per thread)
    for (int c = tid; c < G * LPR; c += 256) {
        const int g = c / LPR, c0 = (c % LPR) * 8;
        const bf16_t* qh = qkv + (int64_t)(kvh * G + g) * DH;
        if (cs) {
            float f[8];
            load_roped<bf16_t>(qh, c0, half_rot, cs, sn, f);
            bf16x8_v r;
#pragma unroll
            for (int e = 0; e < 8; ++e) r[e] = (__bf16)f[e];   // exact: f holds bf16 values
            *reinterpret_cast<bf16x8_v*>(&q_lds[g][c0]) = r;
        } else {
            *reinterpret_cast<uint4*>(&q_lds[g][c0]) = *reinterpret_cast<const uint4*>(qh + c0);
        }
    }
    __syncthreads();

    const int64_t p0 = (int64_t)split * chunk;
    int64_t p1 = p0 + chunk;
    if (p1 > qpos + 1) p1 = qpos + 1;

    // query fragments: column = query head col % G, 8 consecutive d per lane and k-step
    bf16x8_v qf[NK];
#pragma unroll
    for (int kk = 0; kk < NK; ++kk) qf[kk] = *reinterpret_cast<const bf16x8_v*>(&q_lds[col % G][16 * kk + 8 * half]);
    float o[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
        for (int e = 0; e < 8; ++e) o[g][e] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    const int ntiles = p1 > p0 ? (int)((p1 - p0 + 31) / 32) : 0;
    const int iters = (ntiles + 3) / 4;   // uniform over the workgroup
    for (int it = 0; it < iters; ++it) {
        const int buf = it & 1;
        const int64_t kb = p0 + (int64_t)(it * 4 + wave) * 32;
        const bool active = kb < p1;
        uint4 vreg[NV];
        if (active) {
            // rows past the last attended position re-read that position and get probability zero
            const bf16_t* krow = kbase + (kb + col < p1 ? kb + col : p1 - 1) * DH + 8 * half;
            bf16x8_v kf[NK];
#pragma unroll
            for (int kk = 0; kk < NK; ++kk) kf[kk] = *reinterpret_cast<const bf16x8_v*>(krow + 16 * kk);
#pragma unroll
            for (int j = 0; j < NV; ++j) {
                const int64_t key = kb + NV * sub + j;
                vreg[j] = *reinterpret_cast<const uint4*>(vbase + (key < p1 ? key : p1 - 1) * DH + li * 8);
            }
            f32x16_v sc;
#pragma unroll
            for (int v = 0; v < 16; ++v) sc[v] = 0.f;
#pragma unroll
            for (int kk = 0; kk < NK; ++kk) sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[kk], qf[kk], sc, 0, 0, 0);
            float mx = -INFINITY;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int64_t key = kb + 8 * (v >> 2) + (v & 3) + 4 * half;
                const float x = key < p1 ? sc[v] * scale_log2e : -INFINITY;
                sc[v] = x;
                mx = fmaxf(mx, x);
            }
            mx = half_max(mx);
            const float m_new = fmaxf(m_run, mx);   // finite: the tile holds at least one attended key
            const float corr = __builtin_amdgcn_exp2f(m_run - m_new);
            float ls = 0.f;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                sc[v] = __builtin_amdgcn_exp2f(sc[v] - m_new);
                ls += sc[v];
            }
            ls = half_sum(ls);
            l_run = l_run * corr + ls;
            m_run = m_new;
            if (col < G) {
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4)
                    *reinterpret_cast<float4*>(&p_lds[buf][wave][col][8 * q4 + 4 * half]) =
                        make_float4(sc[4 * q4], sc[4 * q4 + 1], sc[4 * q4 + 2], sc[4 * q4 + 3]);
                if (half == 0) corr_lds[buf][wave][col] = corr;
            }
        }
        __syncthreads();
        if (active) {
#pragma unroll
            for (int g = 0; g < G; ++g) {
                const float c = corr_lds[buf][wave][g];
#pragma unroll
                for (int e = 0; e < 8; ++e) o[g][e] *= c;
            }
#pragma unroll
            for (int j = 0; j < NV; ++j) {
                const float vf[8] = {bf16lo(vreg[j].x), bf16hi(vreg[j].x), bf16lo(vreg[j].y), bf16hi(vreg[j].y),
                                     bf16lo(vreg[j].z), bf16hi(vreg[j].z), bf16lo(vreg[j].w), bf16hi(vreg[j].w)};
#pragma unroll
                for (int g = 0; g < G; ++g) {
                    const float pj = p_lds[buf][wave][g][NV * sub + j];
#pragma unroll
                    for (int e = 0; e < 8; ++e) o[g][e] += pj * vf[e];
                }
            }
        }
    }

    // merge the lane-groups of this wave (they share the wave's maximum), then the four waves through LDS
#pragma unroll
    for (int off = LPR; off < 64; off <<= 1)
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
            for (int e = 0; e < 8; ++e) o[g][e] += __shfl_xor(o[g][e], off, 64);
    if (sub == 0) {
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
            for (int e = 0; e < 8; ++e) so[wave][g][li * 8 + e] = o[g][e];
    }
    if (lane < G) { sm[wave][lane] = m_run; sl[wave][lane] = l_run; }
    __syncthreads();
    for (int idx = tid; idx < G * DH; idx += 256) {
        const int g = idx / DH, d = idx % DH;
        const float mn = fmaxf(fmaxf(sm[0][g], sm[1][g]), fmaxf(sm[2][g], sm[3][g]));
        float L = 0.f, O = 0.f;
        if (mn != -INFINITY) {
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const float c = exp2f(sm[w][g] - mn);
                L += sl[w][g] * c;
                O += so[w][g][d] * c;
            }
        }
        const int h = kvh * G + g;
        if (nsplit == 1) {
            stf(ctx, (int64_t)h * DH + d, O / L);
        } else {
            float* rec = ws + ((int64_t)h * nsplit + split) * (DH + 2);
            if (d == 0) { rec[0] = mn * 0.6931471805599453f; rec[1] = L; }
            rec[2 + d] = O;
        }
    }
}

template <typename T>
__global__ void attn_decode_combine_kernel(const float* __restrict__ ws, T* __restrict__ ctx, int dh, int nsplit) {
    // grid (n_q, batch): sequence blockIdx.y owns gridDim.x heads of records and of the context
    ws += (int64_t)blockIdx.y * gridDim.x * nsplit * (dh + 2);
    ctx += (int64_t)blockIdx.y * gridDim.x * dh;
    // per-split weights exp(m_s - max) are computed once into LDS; the slice loads of the output
    // loop are then independent of each other
    __shared__ float wgt[kMaxDecodeSplits];
    __shared__ float red[16];
    const int h = blockIdx.x;
    const float* base = ws + (int64_t)h * nsplit * (dh + 2);
    float mn = -INFINITY;
    for (int s = threadIdx.x; s < nsplit; s += blockDim.x) {
        const float ms = base[(int64_t)s * (dh + 2)];
        wgt[s] = ms;
        mn = fmaxf(mn, ms);
    }
    mn = block_max(mn, red);
    float lsum = 0.f;
    for (int s = threadIdx.x; s < nsplit; s += blockDim.x) {
        const float ms = wgt[s];
        const float c = ms == -INFINITY ? 0.f : expf(ms - mn);
        wgt[s] = c;
        lsum += base[(int64_t)s * (dh + 2) + 1] * c;
    }
    const float L = block_sum(lsum, red);  // also orders the wgt[] writes before the reads below
    for (int d = threadIdx.x; d < dh; d += blockDim.x) {
        float O = 0.f;
#pragma unroll 8
        for (int s = 0; s < nsplit; ++s) O += base[(int64_t)s * (dh + 2) + 2 + d] * wgt[s];
        stf(ctx, (int64_t)h * dh + d, O / L);
    }
}

// Launch geometry shared by attn_decode() and attn_decode_workspace_bytes(): chunks of two
// positions per lane-group, capped at kMaxDecodeSplits splits.
static void decode_geometry(int dtype, int64_t dh, int64_t cap, int* nsplit, int64_t* chunk) {
    const int64_t vec = dtype == 0 ? 4 : 8;
    const int64_t lpr = dh / vec > 0 ? dh / vec : 1;
    const int64_t nstream = 4 * (64 / lpr);
    int64_t c = 2 * nstream;
    if (cdiv(cap, c) > kMaxDecodeSplits) c = cdiv(cdiv(cap, kMaxDecodeSplits), 2 * nstream) * 2 * nstream;
    *chunk = c;
    *nsplit = (int)cdiv(cap, c);
}
size_t attn_decode_workspace_bytes(int64_t n_q, int64_t head_dim, int64_t capacity) {
    int ns0, ns2;
    int64_t c;
    decode_geometry(0, head_dim, capacity, &ns0, &c);
    decode_geometry(2, head_dim, capacity, &ns2, &c);
    const int ns = ns0 > ns2 ? ns0 : ns2;
    return (size_t)n_q * (size_t)ns * (size_t)(head_dim + 2) * sizeof(float);
}

// Matrix-core decode path: bf16, head_dim 64 / 128, group sizes 1, 2, 4, 8 (GPTRS_HIP_MFMA_ATTN=0 turns it off).
static bool attn_decode_mfma_ok(const AttnDecodeArgs& a) {
    static const bool use = [] { const char* e = getenv("GPTRS_HIP_MFMA_ATTN"); return !(e && e[0] == '0'); }();
    if (!use || a.dtype != 2 || a.n_kv <= 0 || a.n_q % a.n_kv != 0) return false;
    if (a.head_dim != 64 && a.head_dim != 128) return false;
    if (a.cos && a.rot_half % 8 != 0) return false;
    const int64_t g = a.n_q / a.n_kv;
    return g == 1 || g == 2 || g == 4 || g == 8;
}

static int attn_decode_mfma(hipStream_t s, const AttnDecodeArgs& a) {
    int nsplit;
    int64_t chunk;
    decode_geometry(a.dtype, a.head_dim, a.capacity, &nsplit, &chunk);   // the workspace holds this many splits
    const int nb = a.batch > 1 ? a.batch : 1;
    // chunks of whole 32-key tiles, never shorter than the workspace geometry's; lengthened until the launch is
    // near four workgroups per CU (each wave then walks several tiles)
    const int64_t step = chunk > 32 ? chunk : 32;
    chunk = step;
    nsplit = (int)cdiv(a.capacity, chunk);
    while (nsplit > 1 && (int64_t)a.n_kv * nb * nsplit > 1024) {
        chunk += step;
        nsplit = (int)cdiv(a.capacity, chunk);
    }
    dim3 grid((unsigned)a.n_kv, (unsigned)nsplit, (unsigned)nb);
    DecodeCaches caches{};
    for (int b = 0; b < nb && b < 16; ++b) { caches.k[b] = a.k_caches[b]; caches.v[b] = a.v_caches[b]; }
    const float sl = a.scale * 1.44269504088896f;
    const int g = (int)(a.n_q / a.n_kv);
#define GPTRS_LAUNCH(DH, G)                                                                                          \
    attn_decode_mfma_kernel<DH, G><<<grid, 256, 0, s>>>((const bf16_t*)a.qkv, (bf16_t*)a.k_cache, (bf16_t*)a.v_cache, \
        a.update_starts, a.query_start, (bf16_t*)a.ctx, (float*)a.ws, (int)a.n_q, (int)a.n_kv, a.capacity, sl, chunk, \
        nsplit, (const bf16_t*)a.cos, (const bf16_t*)a.sin, (int)a.rot_half, a.batch > 1 ? 1 : 0, caches)
#define GPTRS_LAUNCH_G(DH)                                                                                           \
    switch (g) {                                                                                                     \
        case 1: GPTRS_LAUNCH(DH, 1); break;                                                                          \
        case 2: GPTRS_LAUNCH(DH, 2); break;                                                                          \
        case 4: GPTRS_LAUNCH(DH, 4); break;                                                                          \
        default: GPTRS_LAUNCH(DH, 8); break;                                                                         \
    }
    if (a.head_dim == 64) { GPTRS_LAUNCH_G(64) } else { GPTRS_LAUNCH_G(128) }
#undef GPTRS_LAUNCH_G
#undef GPTRS_LAUNCH
    if (nsplit > 1) {
        const int block = a.head_dim <= 64 ? 64 : 128;
        attn_decode_combine_kernel<bf16_t><<<dim3((unsigned)a.n_q, (unsigned)nb), block, 0, s>>>((const float*)a.ws, (bf16_t*)a.ctx, (int)a.head_dim, nsplit);
    }
    return nsplit > 1 ? 2 : 1;
}

template <typename T>
static int attn_decode_t(hipStream_t s, const AttnDecodeArgs& a) {
    int nsplit;
    int64_t chunk;
    decode_geometry(a.dtype, a.head_dim, a.capacity, &nsplit, &chunk);
    const int nb = a.batch > 1 ? a.batch : 1;
    // a batch multiplies the workgroups: longer chunks keep the launch near six workgroups per CU, so the fixed cost
    // of a workgroup (query load, state merges, record) is spread over more positions (fewer splits than the
    // workspace was sized for is always safe)
    const int64_t step = chunk;
    while (nsplit > 1 && (int64_t)a.n_kv * nb * nsplit > 1536) {
        chunk += step;
        nsplit = (int)cdiv(a.capacity, chunk);
    }
    // a short cache is one chunk: the workgroup walks only the positions that are valid (its loop ends at the query
    // position, at most four rounds of loads), stores the context row itself, and the launch of the combine kernel is
    // saved (GPT-2 generate 64 at capacity 128: 1910 -> 1999 tokens/s; at capacity 256 the longer walk costs what the
    // launch saves)
    if (a.capacity <= 128) { chunk = a.capacity; nsplit = 1; }
    dim3 grid((unsigned)a.n_kv, (unsigned)nsplit, (unsigned)nb);
    const int g = (int)(a.n_q / a.n_kv);
    DecodeCaches caches{};
    for (int b = 0; b < nb && b < 16; ++b) { caches.k[b] = a.k_caches[b]; caches.v[b] = a.v_caches[b]; }
#define GPTRS_LAUNCH(G)                                                                                          \
    attn_decode_kernel<T, G><<<grid, 256, 0, s>>>((const T*)a.qkv, (T*)a.k_cache, (T*)a.v_cache, a.update_starts,    \
        a.query_start, (T*)a.ctx, (float*)a.ws, (int)a.n_q, (int)a.n_kv, (int)a.head_dim, a.capacity, a.scale, chunk, nsplit, \
        (const T*)a.cos, (const T*)a.sin, (int)a.rot_half, a.batch > 1 ? 1 : 0, caches)
    switch (g) {
        case 1: GPTRS_LAUNCH(1); break;
        case 2: GPTRS_LAUNCH(2); break;
        case 4: GPTRS_LAUNCH(4); break;
        default: GPTRS_LAUNCH(8); break;
    }
#undef GPTRS_LAUNCH
    if (nsplit > 1) {
        const int block = a.head_dim <= 64 ? 64 : (a.head_dim <= 128 ? 128 : 256);
        attn_decode_combine_kernel<T><<<dim3((unsigned)a.n_q, (unsigned)nb), block, 0, s>>>((const float*)a.ws, (T*)a.ctx, (int)a.head_dim, nsplit);
    }
    return nsplit > 1 ? 2 : 1;
}
int attn_decode(hipStream_t s, const AttnDecodeArgs& a) {
    if (attn_decode_mfma_ok(a)) return attn_decode_mfma(s, a);
    return a.dtype == 0 ? attn_decode_t<float>(s, a) : attn_decode_t<bf16_t>(s, a);
}

// ------------------------------------------------------------------------------ prefill
// grid (ceil(T/4), n_q), 256 threads: one wave per query row.  Keys are visited 64 at a time
// (one per lane) with an online softmax; the P.V update then walks the chunk with the lanes
// spread over head_dim so V rows are read coalesced.
template <typename T>
__global__ __launch_bounds__(256) void attn_prefill_kernel(const T* __restrict__ qkv, T* __restrict__ ctx, int64_t t,
                                                           int n_q, int n_kv, int dh, float scale) {
    __shared__ float qsm[4][256];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t i = (int64_t)blockIdx.x * 4 + wave;
    const int h = blockIdx.y;
    const int kvh = h / (n_q / n_kv);
    const int64_t P = (int64_t)(n_q + 2 * n_kv) * dh;
    const int64_t koff = (int64_t)n_q * dh + (int64_t)kvh * dh;
    const int64_t voff = (int64_t)(n_q + n_kv) * dh + (int64_t)kvh * dh;
    if (i < t)
        for (int d = lane; d < dh; d += 64) qsm[wave][d] = ldf(qkv, i * P + (int64_t)h * dh + d);
    __syncthreads();
    if (i >= t) return;
    float m = -INFINITY, l = 0.f;
    float o[4] = {0.f, 0.f, 0.f, 0.f};
    for (int64_t j0 = 0; j0 <= i; j0 += 64) {
        const int64_t j = j0 + lane;
        float s = -INFINITY;
        if (j <= i) {
            const T* kr = qkv + j * P + koff;
            float acc = 0.f;
            for (int d = 0; d < dh; ++d) acc += qsm[wave][d] * ldf(kr, d);
            s = acc * scale;
        }
        const float mn = fmaxf(m, wave_max(s));
        const float corr = expf(m - mn);
        const float pe = j <= i ? expf(s - mn) : 0.f;
        l = l * corr + wave_sum(pe);
#pragma unroll
        for (int c = 0; c < 4; ++c) o[c] *= corr;
        const int cnt = (int)((i - j0 + 1) < 64 ? (i - j0 + 1) : 64);
        for (int jj = 0; jj < cnt; ++jj) {
            const float pj = __shfl(pe, jj, 64);
            const T* vr = qkv + (j0 + jj) * P + voff;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int d = lane + 64 * c;
                if (d < dh) o[c] += pj * ldf(vr, d);
            }
        }
        m = mn;
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const int d = lane + 64 * c;
        if (d < dh) stf(ctx, i * (int64_t)n_q * dh + (int64_t)h * dh + d, o[c] / l);
    }
}
// bf16 prefill attention on the matrix cores (flash-attention style, causal, grouped-query).
//
// A workgroup (4 waves) serves one kv head and up to 4 query heads of its group over 32 query rows each, so a key /
// value tile staged in LDS is used by every query head that shares it and all waves see the same causal range.  Per
// tile of 32 keys a wave computes with v_mfma_f32_32x32x16_bf16
//   S^T[key, q] = K[key, :] . Q[q, :]      (A = K rows from LDS, B = Q fragments kept in registers)
//   O^T[d, q]  += V^T[d, key] . P^T[key, q] (A = V^T from LDS, B = the probabilities just computed, from registers)
// Both products are taken transposed so that a lane always owns ONE query (column lane % 32): the 16 scores a lane
// holds belong to its query, the online-softmax state (running maximum and sum, in the log2 domain) is a per-lane
// scalar, the rescaling of O^T is a per-lane multiply, and P^T needs no cross-lane movement to become the B operand:
// the k-slots of the second product are simply numbered in the order the lane holds its keys, and V^T is written to
// LDS in that order (key bits 2 and 3 swapped).
// KG = 2: the workgroup has two groups of four waves; both serve the same queries, group g takes the key tiles
// 2 s + g (it stages them itself, into its own LDS buffers), and the two online-softmax states meet through LDS at the
// end.  A row tile then takes half as many steps, and a SIMD holds two waves whose matrix and vector phases overlap
// (the launch has one wave-sized task per SIMD otherwise).
template <int DH, int KG>
__global__ __launch_bounds__(256 * KG, 2 / KG) void attn_prefill_mfma_kernel(const bf16_t* __restrict__ qkv, bf16_t* __restrict__ ctx, int T,
                                                                int n_q, int n_kv, float scale_log2e) {
    constexpr int KT = 32;            // keys per tile
    constexpr int KS = DH + 8;        // K tile row stride in elements (16 bytes of padding)
    // V^T rows: stride VS elements, row d starts 8 * ((d / 8) % 8) elements in.  Two access patterns must spread over
    // the 32 banks: a fragment read (8 lanes = 8 consecutive rows, 16 bytes each) wants the row stride to be an odd
    // multiple of 16 bytes modulo 128 (104 elements = 208 bytes: rows land 20 banks apart), and the scatter of one key's
    // d-chunks (16 lanes, 8 rows apart, same position) would hit a single bank whatever the stride (8 rows are a
    // multiple of 128 bytes apart), which the skew spreads over 8 groups of 4 banks.  Measured at 1024 tokens: no skew
    // 88 us per layer, skew with 128-byte rows (reads 8-way conflicting) 68 us.
    // Two key groups: rows of 88 elements (176 bytes: consecutive rows 44 banks apart, so the 8 rows of one d-chunk fall
    // into 8 different groups of 4 banks, and a chunk's first row starts 32 banks from its neighbour's) and a skew of
    // 16 bytes x (chunk / 2): the 16 chunks of one key then scatter into 16 different groups of 4 banks (with 72-element
    // rows and 4 skews they shared 4, an 8-way conflict on every 2-byte store: 2.7 M conflict cycles per launch).
    constexpr int VS = KG == 1 ? 104 : 88;
    constexpr int SKEW = 7;
    constexpr int SKSH = KG == 1 ? 0 : 1;     // the skew index is (chunk >> SKSH) & SKEW
    constexpr int ND = DH / 32;       // 32-row blocks of d in O^T
    constexpr int NK = DH / 16;       // k-steps of the score product
    constexpr int CH = KT * DH / 8;   // 16-byte chunks of a K (or V) tile
    constexpr int CPT = (CH + 255) / 256;
    __shared__ __align__(16) bf16_t ksm_all[KG][2][KT * KS];
    __shared__ __align__(16) bf16_t vsm_all[KG][2][DH * VS];

    const int kg = threadIdx.x / 256;                     // key group of this wave
    const int tid = threadIdx.x % 256, lane = tid & 63, wave = tid >> 6;
    bf16_t (*ksm)[KT * KS] = ksm_all[kg];
    bf16_t (*vsm)[DH * VS] = vsm_all[kg];
    const int col = lane & 31, half = lane >> 5;
    const int G = n_q / n_kv;
    const int gw = G >= 4 ? 4 : G;                 // query heads of the group in this workgroup
    const int rtpb = 4 / gw;                       // 32-row tiles per workgroup
    const int kvh = blockIdx.y;
    const int head = kvh * G + blockIdx.z * gw + wave % gw;
    const int q0 = (blockIdx.x * rtpb + wave / gw) * 32;
    const int64_t P = (int64_t)(n_q + 2 * n_kv) * DH;
    const int64_t koff = (int64_t)n_q * DH + (int64_t)kvh * DH;
    const int64_t voff = (int64_t)(n_q + n_kv) * DH + (int64_t)kvh * DH;
    const int kend = min(T, (blockIdx.x * rtpb + rtpb) * 32);   // keys any row of the workgroup may see
    const int ntiles = (kend + KT - 1) / KT;
    const bool active = q0 < T;
    const int my_tiles = active ? min(ntiles, (q0 + 31) / KT + 1) : 0;   // tiles holding a key <= this wave's last row

    // Q fragments (B operand: column = query, 8 consecutive d per lane and k-step)
    bf16x8_v qf[NK];
    {
        const int row = min(q0 + col, T - 1);
        const bf16_t* qp = qkv + (int64_t)row * P + (int64_t)head * DH + 8 * half;
#pragma unroll
        for (int kk = 0; kk < NK; ++kk) qf[kk] = *reinterpret_cast<const bf16x8_v*>(qp + 16 * kk);
    }
    f32x16_v acc_o[ND];
#pragma unroll
    for (int db = 0; db < ND; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc_o[db][v] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    // native vectors and unconditional loads (the chunk index is clamped instead): with HIP's uint4 struct and a
    // guarded load the compiler keeps these in scratch memory and waits for every load right where it is issued
    typedef uint32_t u32x4_s __attribute__((ext_vector_type(4)));
    u32x4_s kreg[CPT], vreg[CPT];
    auto gload = [&](int t) {
#pragma unroll
        for (int j = 0; j < CPT; ++j) {
            const int c = min(tid + 256 * j, CH - 1);
            const int r = c / (DH / 8), ch = c % (DH / 8);
            const int64_t key = min(t * KT + r, T - 1);
            kreg[j] = *reinterpret_cast<const u32x4_s*>(qkv + key * P + koff + ch * 8);
            vreg[j] = *reinterpret_cast<const u32x4_s*>(qkv + key * P + voff + ch * 8);
        }
    };
    auto lwrite = [&](int buf) {
#pragma unroll
        for (int j = 0; j < CPT; ++j) {
            const int c = tid + 256 * j;
            if (CH % 256 == 0 || c < CH) {
                const int r = c / (DH / 8), ch = c % (DH / 8);
                *reinterpret_cast<u32x4_s*>(&ksm[buf][r * KS + ch * 8]) = kreg[j];
                // key r goes to k-slot position p: bits 2 and 3 of r swapped
                const int pos = (r & 0x13) | ((r & 4) << 1) | ((r & 8) >> 1);
                const uint32_t w0 = vreg[j].x, w1 = vreg[j].y, w2 = vreg[j].z, w3 = vreg[j].w;
                const uint32_t w[4] = {w0, w1, w2, w3};
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    vsm[buf][(ch * 8 + e) * VS + 8 * ((ch >> SKSH) & SKEW) + pos] = (bf16_t)((w[e >> 1] >> ((e & 1) * 16)) & 0xFFFFu);
            }
        }
    };

    // group kg visits tiles kg, kg + KG, ...; the step count is uniform over the workgroup (barriers)
    const int nsteps = (ntiles + KG - 1) / KG;
    if (kg < ntiles) { gload(kg); lwrite(0); }
    // The Q fragments are used here, once, so that they have arrived on EVERY path into the step loop.  A workgroup whose
    // group has no first tile skips the wait above; the compiler then assumes the eight Q loads may still be in flight at
    // the loop's head and puts `s_waitcnt vmcnt(7) .. vmcnt(0)` in front of the eight score MFMAs of every step, which in
    // steady state wait for the tile requested at the top of that same step (37.1 -> 34.5 us per layer at 1024 tokens).
    // Two tiles in flight instead of one (a second register set, roles swapped from step to step) gained nothing more.
#pragma unroll
    for (int kk = 0; kk < NK; ++kk) asm volatile("" : : "v"(qf[kk]));
    __syncthreads();
    for (int st = 0; st < nsteps; ++st) {
        const int buf = st & 1;
        const int t = st * KG + kg;
        if (t + KG < ntiles) gload(t + KG);
        if (t < my_tiles) {
            // scores, transposed: rows = keys of the tile, column = this lane's query
            f32x16_v sc;
#pragma unroll
            for (int v = 0; v < 16; ++v) sc[v] = 0.f;
#pragma unroll
            for (int kk = 0; kk < NK; ++kk) {
                const bf16x8_v kf = *reinterpret_cast<const bf16x8_v*>(&ksm[buf][col * KS + 16 * kk + 8 * half]);
                sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[kk], sc, 0, 0, 0);
            }
            const int qrow = q0 + col;
            const int kbase = t * KT + 4 * half;
            // raw scores: the (positive) scale is applied inside the exponent's fma; only a tile that reaches past the
            // wave's first row holds keys to mask
            if (t * KT + KT - 1 > q0) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int key = kbase + 8 * (v >> 2) + (v & 3);
                    if (key > qrow) sc[v] = -INFINITY;
                }
            }
            float mx = -INFINITY;
#pragma unroll
            for (int v = 0; v < 16; ++v) mx = fmaxf(mx, sc[v]);
            mx = half_max(mx) * scale_log2e;
            // The reference point of the exponentials follows the running maximum lazily: it moves only when the
            // maximum has grown by more than 2^8 (probabilities then reach 2^8 at most, harmless in bf16 / f32, and
            // the quotient O / l does not depend on the reference point).  Most tiles therefore leave O^T unscaled,
            // and a wave skips the 64 multiplies (the accumulators live in AGPRs: 128 more moves) unless a lane moved.
            const bool move = mx > m_run + 8.0f;    // first tile: m_run = -inf, key 0 is visible to every query
            const float m_new = move ? mx : m_run;
            const float corr = move ? __builtin_amdgcn_exp2f(m_run - m_new) : 1.0f;
            float ls = 0.f;
            bf16x8_v pb[2];
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const float pv = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[v], scale_log2e, -m_new));
                ls += pv;
                pb[v >> 3][v & 7] = (__bf16)pv;
            }
            ls = half_sum(ls);
            l_run = l_run * corr + ls;
            m_run = m_new;
            if (__builtin_amdgcn_ballot_w64(move) != 0) {
#pragma unroll
                for (int db = 0; db < ND; ++db)
#pragma unroll
                    for (int v = 0; v < 16; ++v) acc_o[db][v] *= corr;
            }
#pragma unroll
            for (int db = 0; db < ND; ++db) {
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const bf16x8_v vf = *reinterpret_cast<const bf16x8_v*>(&vsm[buf][(db * 32 + col) * VS + 8 * (((db * 4 + (col >> 3)) >> SKSH) & SKEW) + 16 * i + 8 * half]);
                    acc_o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pb[i], acc_o[db], 0, 0, 0);
                }
            }
        }
        if (t + KG < ntiles) lwrite(buf ^ 1);
        __syncthreads();
    }
    if (KG == 2) {
        // merge the two groups' states: O = O0 c0 + O1 c1, l = l0 c0 + l1 c1 with c_g = 2^(m_g - max(m0, m1)); a group
        // that saw no tile has m = -inf, l = 0, O = 0 and drops out.  The tiles in LDS are dead (the loop ended on a
        // barrier); the exchange area is 66 floats per lane of the second group.
        float* xch = reinterpret_cast<float*>(&vsm_all[0][0][0]) + (wave * 64 + lane);
        static_assert(KG == 1 || (ND * 16 + 2) * 256 * 4 <= (int)sizeof(vsm_all), "exchange area fits the V buffers");
        if (kg == 1) {
#pragma unroll
            for (int db = 0; db < ND; ++db)
#pragma unroll
                for (int v = 0; v < 16; ++v) xch[(db * 16 + v) * 256] = acc_o[db][v];
            xch[(ND * 16) * 256] = m_run;
            xch[(ND * 16 + 1) * 256] = l_run;
        }
        __syncthreads();
        if (kg == 1) return;
        const float m1 = xch[(ND * 16) * 256], l1 = xch[(ND * 16 + 1) * 256];
        const float mm = fmaxf(m_run, m1);
        const float c0 = __builtin_amdgcn_exp2f(m_run - mm), c1 = __builtin_amdgcn_exp2f(m1 - mm);
        l_run = l_run * c0 + l1 * c1;
#pragma unroll
        for (int db = 0; db < ND; ++db)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc_o[db][v] = acc_o[db][v] * c0 + xch[(db * 16 + v) * 256] * c1;
    }
    if (active && q0 + col < T) {
        const float inv = 1.0f / l_run;
        bf16_t* op = ctx + (int64_t)(q0 + col) * n_q * DH + (int64_t)head * DH;
#pragma unroll
        for (int db = 0; db < ND; ++db)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const int d = db * 32 + 8 * g4 + 4 * half;
                const uint32_t lo = pack_bf16x2(acc_o[db][4 * g4 + 0] * inv, acc_o[db][4 * g4 + 1] * inv);
                const uint32_t hi = pack_bf16x2(acc_o[db][4 * g4 + 2] * inv, acc_o[db][4 * g4 + 3] * inv);
                *reinterpret_cast<uint2*>(op + d) = make_uint2(lo, hi);
            }
    }
}

// The same kernel in f32 on v_mfma_f32_32x32x2_f32: a 16-byte fragment holds 4 consecutive d (scores) or 4 consecutive
// keys (P.V), each fragment feeds four K = 2 products, and the probabilities stay f32.  V^T sits in LDS in plain key
// order: the keys a lane holds of its query in score registers 4 i .. 4 i + 3 are 8 i + 4 (lane / 32) + 0..3, exactly
// what fragment i of the second product covers.
typedef float f32x4_v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ f32x16_v mma_f32x4(const f32x4_v& a, const f32x4_v& b, f32x16_v c) {
#pragma unroll
    for (int e = 0; e < 4; ++e) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], b[e], c, 0, 0, 0);
    return c;
}

template <int DH>
__global__ __launch_bounds__(256, 2) void attn_prefill_mfma_f32_kernel(const float* __restrict__ qkv, float* __restrict__ ctx, int T,
                                                                    int n_q, int n_kv, float scale_log2e) {
    constexpr int KT = 32;            // keys per tile
    constexpr int KS = DH + 4;        // K tile row stride in elements (16 bytes of padding)
    // V^T row stride in elements; row d starts 4 * ((d / 4) % 8) elements in, which spreads the lanes that scatter one
    // key's d-chunks over the banks (as in the bf16 kernel)
    constexpr int VS = KT + 4 + 28;
    constexpr int ND = DH / 32;       // 32-row blocks of d in O^T
    constexpr int NK = DH / 8;        // k-steps of the score product (8 d each)
    constexpr int CH = KT * DH / 4;   // 16-byte chunks of a K (or V) tile
    constexpr int CPT = (CH + 255) / 256;
    __shared__ __align__(16) float ksm[2][KT * KS];
    __shared__ __align__(16) float vsm[2][DH * VS];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, half = lane >> 5;
    const int G = n_q / n_kv;
    const int gw = G >= 4 ? 4 : G;
    const int rtpb = 4 / gw;
    const int kvh = blockIdx.y;
    const int head = kvh * G + blockIdx.z * gw + wave % gw;
    const int q0 = (blockIdx.x * rtpb + wave / gw) * 32;
    const int64_t P = (int64_t)(n_q + 2 * n_kv) * DH;
    const int64_t koff = (int64_t)n_q * DH + (int64_t)kvh * DH;
    const int64_t voff = (int64_t)(n_q + n_kv) * DH + (int64_t)kvh * DH;
    const int kend = min(T, (blockIdx.x * rtpb + rtpb) * 32);
    const int ntiles = (kend + KT - 1) / KT;
    const bool active = q0 < T;
    const int my_tiles = active ? min(ntiles, (q0 + 31) / KT + 1) : 0;

    f32x4_v qf[NK];
    {
        const int row = min(q0 + col, T - 1);
        const float* qp = qkv + (int64_t)row * P + (int64_t)head * DH + 4 * half;
#pragma unroll
        for (int kk = 0; kk < NK; ++kk) qf[kk] = *reinterpret_cast<const f32x4_v*>(qp + 8 * kk);
    }
    f32x16_v acc_o[ND];
#pragma unroll
    for (int db = 0; db < ND; ++db)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc_o[db][v] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    f32x4_v kreg[CPT], vreg[CPT];
    auto gload = [&](int t) {
#pragma unroll
        for (int j = 0; j < CPT; ++j) {
            const int c = min(tid + 256 * j, CH - 1);   // unconditional loads: see the bf16 kernel
            const int r = c / (DH / 4), ch = c % (DH / 4);
            const int64_t key = min(t * KT + r, T - 1);
            kreg[j] = *reinterpret_cast<const f32x4_v*>(qkv + key * P + koff + ch * 4);
            vreg[j] = *reinterpret_cast<const f32x4_v*>(qkv + key * P + voff + ch * 4);
        }
    };
    auto lwrite = [&](int buf) {
#pragma unroll
        for (int j = 0; j < CPT; ++j) {
            const int c = tid + 256 * j;
            if (CH % 256 == 0 || c < CH) {
                const int r = c / (DH / 4), ch = c % (DH / 4);
                *reinterpret_cast<f32x4_v*>(&ksm[buf][r * KS + ch * 4]) = kreg[j];
#pragma unroll
                for (int e = 0; e < 4; ++e) vsm[buf][(ch * 4 + e) * VS + 4 * (ch & 7) + r] = vreg[j][e];
            }
        }
    };

    gload(0);
    lwrite(0);
    // the Q fragments have arrived before the step loop on every path (see attn_prefill_mfma_kernel)
#pragma unroll
    for (int kk = 0; kk < NK; ++kk) asm volatile("" : : "v"(qf[kk]));
    __syncthreads();
    for (int t = 0; t < ntiles; ++t) {
        const int buf = t & 1;
        if (t + 1 < ntiles) gload(t + 1);
        if (t < my_tiles) {
            f32x16_v sc;
#pragma unroll
            for (int v = 0; v < 16; ++v) sc[v] = 0.f;
#pragma unroll
            for (int kk = 0; kk < NK; ++kk) {
                const f32x4_v kf = *reinterpret_cast<const f32x4_v*>(&ksm[buf][col * KS + 8 * kk + 4 * half]);
                sc = mma_f32x4(kf, qf[kk], sc);
            }
            const int qrow = q0 + col;
            const int kbase = t * KT + 4 * half;
            if (t * KT + KT - 1 > q0) {   // only a tile that reaches past the wave's first row holds keys to mask
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int key = kbase + 8 * (v >> 2) + (v & 3);
                    if (key > qrow) sc[v] = -INFINITY;
                }
            }
            float mx = -INFINITY;
#pragma unroll
            for (int v = 0; v < 16; ++v) mx = fmaxf(mx, sc[v]);
            mx = half_max(mx) * scale_log2e;
            // lazy reference point and wave-wide skip of the rescaling, as in the bf16 kernel
            const bool move = mx > m_run + 8.0f;
            const float m_new = move ? mx : m_run;
            const float corr = move ? __builtin_amdgcn_exp2f(m_run - m_new) : 1.0f;
            float ls = 0.f;
            f32x4_v pf[4];
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const float pv = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[v], scale_log2e, -m_new));
                ls += pv;
                pf[v >> 2][v & 3] = pv;
            }
            ls = half_sum(ls);
            l_run = l_run * corr + ls;
            m_run = m_new;
            if (__builtin_amdgcn_ballot_w64(move) != 0) {
#pragma unroll
                for (int db = 0; db < ND; ++db)
#pragma unroll
                    for (int v = 0; v < 16; ++v) acc_o[db][v] *= corr;
            }
#pragma unroll
            for (int db = 0; db < ND; ++db) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const f32x4_v vf = *reinterpret_cast<const f32x4_v*>(&vsm[buf][(db * 32 + col) * VS + 4 * ((col >> 2) & 7) + 8 * i + 4 * half]);
                    acc_o[db] = mma_f32x4(vf, pf[i], acc_o[db]);
                }
            }
        }
        if (t + 1 < ntiles) lwrite(buf ^ 1);
        __syncthreads();
    }
    if (active && q0 + col < T) {
        const float inv = 1.0f / l_run;
        float* op = ctx + (int64_t)(q0 + col) * n_q * DH + (int64_t)head * DH;
#pragma unroll
        for (int db = 0; db < ND; ++db)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const int d = db * 32 + 8 * g4 + 4 * half;
                *reinterpret_cast<float4*>(op + d) = make_float4(acc_o[db][4 * g4] * inv, acc_o[db][4 * g4 + 1] * inv,
                                                                 acc_o[db][4 * g4 + 2] * inv, acc_o[db][4 * g4 + 3] * inv);
            }
    }
}

static bool attn_prefill_mfma_ok(const AttnPrefillArgs& a) {
    if ((a.dtype != 2 && a.dtype != 0) || a.n_kv <= 0 || a.n_q % a.n_kv != 0 || a.t >= (1ll << 30)) return false;
    if (a.head_dim != 32 && a.head_dim != 64 && a.head_dim != 128) return false;
    const int64_t g = a.n_q / a.n_kv;
    return g == 1 || g == 2 || g % 4 == 0;
}

void attn_prefill(hipStream_t s, const AttnPrefillArgs& a) {
    if (a.t <= 0) return;
    static const bool use_mfma = [] { const char* e = getenv("GPTRS_HIP_MFMA_ATTN"); return !(e && e[0] == '0'); }();
    if (use_mfma && attn_prefill_mfma_ok(a)) {
        const int g = (int)(a.n_q / a.n_kv), gw = g >= 4 ? 4 : g;
        dim3 grid((unsigned)cdiv(cdiv(a.t, 32), 4 / gw), (unsigned)a.n_kv, (unsigned)(g >= 4 ? g / 4 : 1));
        const float sl = a.scale * 1.44269504088896f;
        if (a.dtype == 0) {
            if (a.head_dim == 32) attn_prefill_mfma_f32_kernel<32><<<grid, 256, 0, s>>>((const float*)a.qkv, (float*)a.ctx, (int)a.t, (int)a.n_q, (int)a.n_kv, sl);
            else if (a.head_dim == 64) attn_prefill_mfma_f32_kernel<64><<<grid, 256, 0, s>>>((const float*)a.qkv, (float*)a.ctx, (int)a.t, (int)a.n_q, (int)a.n_kv, sl);
            else attn_prefill_mfma_f32_kernel<128><<<grid, 256, 0, s>>>((const float*)a.qkv, (float*)a.ctx, (int)a.t, (int)a.n_q, (int)a.n_kv, sl);
            return;
        }
        // two key groups per workgroup once the launch is smaller than three workgroups per CU and rows are long
        // enough to split
        static const bool allow_kg = [] { const char* e = getenv("GPTRS_HIP_ATTN_KEYGROUPS"); return !(e && e[0] == '0'); }();
        const bool kg2 = allow_kg && a.t >= 128 && (int64_t)grid.x * grid.y * grid.z < 768;
#define GPTRS_PREFILL(DHV)                                                                                                   \
        do {                                                                                                                 \
            if (kg2) attn_prefill_mfma_kernel<DHV, 2><<<grid, 512, 0, s>>>((const bf16_t*)a.qkv, (bf16_t*)a.ctx, (int)a.t, (int)a.n_q, (int)a.n_kv, sl); \
            else attn_prefill_mfma_kernel<DHV, 1><<<grid, 256, 0, s>>>((const bf16_t*)a.qkv, (bf16_t*)a.ctx, (int)a.t, (int)a.n_q, (int)a.n_kv, sl);     \
        } while (0)
        if (a.head_dim == 32) GPTRS_PREFILL(32);
        else if (a.head_dim == 64) GPTRS_PREFILL(64);
        else GPTRS_PREFILL(128);
#undef GPTRS_PREFILL
        return;
    }
    dim3 grid((unsigned)cdiv(a.t, 4), (unsigned)a.n_q);
    if (a.dtype == 0)
        attn_prefill_kernel<float><<<grid, 256, 0, s>>>((const float*)a.qkv, (float*)a.ctx, a.t, (int)a.n_q, (int)a.n_kv, (int)a.head_dim, a.scale);
    else
        attn_prefill_kernel<bf16_t><<<grid, 256, 0, s>>>((const bf16_t*)a.qkv, (bf16_t*)a.ctx, a.t, (int)a.n_q, (int)a.n_kv, (int)a.head_dim, a.scale);
}

// ------------------------------------------------------------------------------ attention over a growing cache
// k_all / v_all [n_kv, L, dh], L = C + T: positions < C from the caches, the rest from the K / V blocks of packed qkv
template <typename T>
__global__ __launch_bounds__(256) void attn_concat_kv_kernel(const T* __restrict__ qkv, const T* __restrict__ kc, const T* __restrict__ vc,
                                                             T* __restrict__ k_all, T* __restrict__ v_all, int64_t t, int64_t c,
                                                             int n_q, int n_kv, int dh) {
    const int64_t L = c + t, total = (int64_t)n_kv * L * dh;
    const int64_t P = (int64_t)(n_q + 2 * n_kv) * dh;
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += (int64_t)gridDim.x * 256) {
        const int d = (int)(e % dh);
        const int64_t pos = (e / dh) % L;
        const int h = (int)(e / ((int64_t)dh * L));
        if (pos < c) {
            const int64_t src = ((int64_t)h * c + pos) * dh + d;
            k_all[e] = kc[src];
            v_all[e] = vc[src];
        } else {
            const int64_t row = (pos - c) * P + (int64_t)h * dh + d;
            k_all[e] = qkv[row + (int64_t)n_q * dh];
            v_all[e] = qkv[row + (int64_t)(n_q + n_kv) * dh];
        }
    }
}
// grid (ceil(T/4), n_q), 256 threads: one wave per query row, as attn_prefill_kernel, over keys 0 .. C + i of the
// combined caches
template <typename T>
__global__ __launch_bounds__(256) void attn_concat_kernel(const T* __restrict__ qkv, const T* __restrict__ k_all, const T* __restrict__ v_all,
                                                          T* __restrict__ ctx, int64_t t, int64_t c, int n_q, int n_kv, int dh, float scale) {
    __shared__ float qsm[4][256];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t i = (int64_t)blockIdx.x * 4 + wave;
    const int h = blockIdx.y;
    const int kvh = h / (n_q / n_kv);
    const int64_t P = (int64_t)(n_q + 2 * n_kv) * dh, L = c + t;
    const T* kb = k_all + (int64_t)kvh * L * dh;
    const T* vb = v_all + (int64_t)kvh * L * dh;
    if (i < t)
        for (int d = lane; d < dh; d += 64) qsm[wave][d] = ldf(qkv, i * P + (int64_t)h * dh + d);
    __syncthreads();
    if (i >= t) return;
    const int64_t last = c + i;   // the row's own position
    float m = -INFINITY, l = 0.f;
    float o[4] = {0.f, 0.f, 0.f, 0.f};
    for (int64_t j0 = 0; j0 <= last; j0 += 64) {
        const int64_t j = j0 + lane;
        float s = -INFINITY;
        if (j <= last) {
            const T* kr = kb + j * dh;
            float acc = 0.f;
            for (int d = 0; d < dh; ++d) acc += qsm[wave][d] * ldf(kr, d);
            s = acc * scale;
        }
        const float mn = fmaxf(m, wave_max(s));
        const float corr = expf(m - mn);
        const float pe = j <= last ? expf(s - mn) : 0.f;
        l = l * corr + wave_sum(pe);
#pragma unroll
        for (int cc = 0; cc < 4; ++cc) o[cc] *= corr;
        const int cnt = (int)((last - j0 + 1) < 64 ? (last - j0 + 1) : 64);
        for (int jj = 0; jj < cnt; ++jj) {
            const float pj = __shfl(pe, jj, 64);
            const T* vr = vb + (j0 + jj) * dh;
#pragma unroll
            for (int cc = 0; cc < 4; ++cc) {
                const int d = lane + 64 * cc;
                if (d < dh) o[cc] += pj * ldf(vr, d);
            }
        }
        m = mn;
    }
#pragma unroll
    for (int cc = 0; cc < 4; ++cc) {
        const int d = lane + 64 * cc;
        if (d < dh) stf(ctx, i * (int64_t)n_q * dh + (int64_t)h * dh + d, o[cc] / l);
    }
}
template <typename T>
static void attn_concat_t(hipStream_t s, const AttnConcatArgs& a) {
    const int64_t total = a.n_kv * (a.cache_len + a.t) * a.head_dim;
    const unsigned g = (unsigned)std::min<int64_t>(cdiv(total, 256), 4096);
    attn_concat_kv_kernel<T><<<g, 256, 0, s>>>((const T*)a.qkv, (const T*)a.k_cache, (const T*)a.v_cache, (T*)a.k_all, (T*)a.v_all, a.t,
                                               a.cache_len, (int)a.n_q, (int)a.n_kv, (int)a.head_dim);
    dim3 grid((unsigned)cdiv(a.t, 4), (unsigned)a.n_q);
    attn_concat_kernel<T><<<grid, 256, 0, s>>>((const T*)a.qkv, (const T*)a.k_all, (const T*)a.v_all, (T*)a.ctx, a.t, a.cache_len,
                                               (int)a.n_q, (int)a.n_kv, (int)a.head_dim, a.scale);
}
void attn_concat(hipStream_t s, const AttnConcatArgs& a) {
    if (a.t <= 0) return;
    if (a.dtype == 0) attn_concat_t<float>(s, a);
    else attn_concat_t<bf16_t>(s, a);
}

}  // namespace k
}  // namespace gptrs
