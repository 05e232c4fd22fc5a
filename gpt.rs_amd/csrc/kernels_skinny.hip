// Batched-decode linear layers (2 <= M <= 16 rows, bf16 or f32) on the matrix cores.
//
// With a handful of rows a linear layer is still one pass over the weights, i.e. bound by HBM, but the
// per-element work of a vector GEMV grows with M (M multiply-adds per weight element plus the activation reads)
// until the vector ALUs, not memory, set the pace.  One v_mfma_f32_16x16x32_bf16 multiplies 16 rows by a
// 32 x 16 block of W at a cost that does not depend on M, so the kernel below only has to stream W.
//
// Weights are read from a derived copy Ws[tile][K/8][16 columns][8 k] (tile = 16 output columns): the 64 lanes of
// a wave fetch 32 consecutive k of the tile's 16 columns as ONE contiguous KiB in exactly the B-operand layout
// (lane = 16 * k-group + column holds 8 consecutive k of its column).  A workgroup owns one tile; its 4 waves take
// the 32-k steps round-robin (so the workgroup reads 4 consecutive KiB per round) and add their partial products
// through LDS.  The A operand (lane = 16 * k-group + row) comes straight from x, which is small and stays in L2.
// DUAL computes silu(x.W) * (x.W2) (ops/functional/activation.rs:141-162) from two weight copies.
// f32 takes the same route with 4 k per 16-byte lane word (Ws[tile][K/4][16][4], 16-k steps) on four
// v_mfma_f32_16x16x4_f32 per word.
//
// Weight-only quantised layers (skinny_gemm_quant_kernel<QF, DUAL>) stream the CODES: a lane's 16-byte word holds 16
// int8 codes (k = 64 S + 16 kg + 0..15 of its column: two MFMA steps) or 32 int4 codes (k = 128 Q + 32 kg + 0..31: four
// steps, exactly one scale group), stored biased (+128 / +8) so the unsigned-byte converts apply; the biased codes are
// exact in bf16 and go to the matrix cores as they are, and a second MFMA per step against a column of ones yields
// sum_k x[row, k], which takes the bias out again (x.(q + b) - b.sum x).  int8 scales (per column) are applied in the
// epilogue, int4 group scales when a group's sums are added to the running total.
//
// A layer with few tiles (N = 3072 has 192, fewer than there are CUs) is split along K over gridDim.y workgroups per
// tile so the whole chip streams: each writes its 16 x 16 partial sums to a workspace and takes a ticket; the
// workgroup that draws the last ticket of a tile adds the partials in split order (so the result does not depend on
// which one that is), applies the epilogue and resets the ticket for the next launch.
#include "kernels.hpp"
#include "device_utils.hpp"

namespace gptrs {
namespace k {

namespace {

typedef __bf16 bf16x8_s __attribute__((ext_vector_type(8)));
typedef float f32x4_s __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_s __attribute__((ext_vector_type(4)));

inline int64_t cdiv_s(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Element types: KPC = k per 16-byte lane word; a step of the K loop is 4 k-groups x KPC (32 k of bf16, 16 k of f32).
// f32 runs on v_mfma_f32_16x16x4_f32: element e of both words is k = 4 * k-group + e of the step.
template <typename T> struct SkinnyT;
template <> struct SkinnyT<bf16_t> {
    static constexpr int KPC = 8;
    static __device__ __forceinline__ f32x4_s mma(const u32x4_s& a, const u32x4_s& b, f32x4_s c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_s, a), __builtin_bit_cast(bf16x8_s, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ float ld(const bf16_t* p, int64_t i) { return bf16_to_f32(p[i]); }
    static __device__ __forceinline__ void st(bf16_t* p, int64_t i, float v) { p[i] = f32_to_bf16(v); }
};
template <> struct SkinnyT<float> {
    static constexpr int KPC = 4;
    static __device__ __forceinline__ f32x4_s mma(const u32x4_s& a, const u32x4_s& b, f32x4_s c) {
        const f32x4_s af = __builtin_bit_cast(f32x4_s, a), bf = __builtin_bit_cast(f32x4_s, b);
#pragma unroll
        for (int e = 0; e < 4; ++e) c = __builtin_amdgcn_mfma_f32_16x16x4f32(af[e], bf[e], c, 0, 0, 0);
        return c;
    }
    static __device__ __forceinline__ float ld(const float* p, int64_t i) { return p[i]; }
    static __device__ __forceinline__ void st(float* p, int64_t i, float v) { p[i] = v; }
};

// Ws[tile][kb][c][i] = W[KPC kb + i][16 tile + c], zero outside [K) x [N); one thread per 16-byte group
template <typename T>
__global__ __launch_bounds__(256) void skinny_pack_kernel(const T* __restrict__ w, T* __restrict__ out, int64_t K, int64_t N,
                                                          int64_t KB, int64_t ntiles) {
    constexpr int KPC = SkinnyT<T>::KPC;
    const int64_t total = ntiles * KB * 16;
    for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < total; g += (int64_t)gridDim.x * blockDim.x) {
        const int c = (int)(g & 15);
        const int64_t kb = (g >> 4) % KB, tile = (g >> 4) / KB;
        const int64_t col = tile * 16 + c;
        alignas(16) T r[KPC];
#pragma unroll
        for (int i = 0; i < KPC; ++i) {
            const int64_t kx = kb * KPC + i;
            r[i] = (col < N && kx < K) ? w[kx * N + col] : T(0);
        }
        *reinterpret_cast<uint4*>(out + g * KPC) = *reinterpret_cast<const uint4*>(r);
    }
}

__device__ __forceinline__ float skinny_finish(float v, float v2, bool dual, int act, float bias, bool has_res, float res) {
    if (dual) v = (v / (1.0f + expf(v * -1.0f))) * v2;              // activation.rs:141-162
    v += bias;                                                      // tensor_ops.rs:42-56
    if (act == 1) v = (v * 0.5f) * (erff(v / 1.41421354f) + 1.0f);  // activation.rs:96-113
    if (has_res) v += res;
    return v;
}

template <typename T, bool DUAL>
__global__ __launch_bounds__(256) void skinny_gemm_kernel(const T* __restrict__ x, const T* __restrict__ ws,
                                                          const T* __restrict__ ws2, const T* __restrict__ bias,
                                                          const T* __restrict__ residual, T* __restrict__ y, int M, int K,
                                                          int N, int act, float* __restrict__ part, unsigned* __restrict__ tickets,
                                                          int out_f32) {
    constexpr int U = 4;                         // steps per wave and round, all requested before the first is used
    constexpr int KPC = SkinnyT<T>::KPC, KSTEP = 4 * KPC;
    __shared__ float red[4][DUAL ? 2 : 1][64][4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int c = lane & 15, kg = lane >> 4;     // B: column c, k-group kg; A: row c, k-group kg
    const int tile = blockIdx.x;
    const int ksplit = gridDim.y, ks = blockIdx.y;
    const int s_begin = (int)((int64_t)(K / KSTEP) * ks / ksplit), nsteps = (int)((int64_t)(K / KSTEP) * (ks + 1) / ksplit);
    const u32x4_s* bsrc = reinterpret_cast<const u32x4_s*>(ws) + (int64_t)tile * (K / KPC) * 16 + lane;
    const u32x4_s* bsrc2 = DUAL ? reinterpret_cast<const u32x4_s*>(ws2) + (int64_t)tile * (K / KPC) * 16 + lane : nullptr;
    const int arow = c < M ? c : M - 1;          // rows beyond M re-read the last one; their products are never stored
    const u32x4_s* asrc = reinterpret_cast<const u32x4_s*>(x + (int64_t)arow * K + KPC * kg);

    f32x4_s acc = {0.f, 0.f, 0.f, 0.f}, acc2 = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = s_begin + wave; s0 < nsteps; s0 += 4 * U) {
        u32x4_s b[U], b2[DUAL ? U : 1], a[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int s = s0 + 4 * u < nsteps ? s0 + 4 * u : s0;   // a step past the end repeats the first, weight zero below
            b[u] = bsrc[(int64_t)s * 64];
            if (DUAL) b2[u] = bsrc2[(int64_t)s * 64];
            a[u] = asrc[s * 4];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (s0 + 4 * u < nsteps) {
                acc = SkinnyT<T>::mma(a[u], b[u], acc);
                if (DUAL) acc2 = SkinnyT<T>::mma(a[u], b2[DUAL ? u : 0], acc2);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        red[wave][0][lane][i] = acc[i];
        if (DUAL) red[wave][DUAL ? 1 : 0][lane][i] = acc2[i];
    }
    __syncthreads();
    if (wave != 0) return;
    constexpr int NP = DUAL ? 2 : 1;
    float g[4], up[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        g[i] = up[i] = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            g[i] += red[w][0][lane][i];
            if (DUAL) up[i] += red[w][DUAL ? 1 : 0][lane][i];
        }
    }
    if (ksplit > 1) {
        // partials and tickets cross workgroups through device-scope accesses only (coherent across the L2s of the
        // XCDs without cache maintenance): stores acknowledged, then the ticket
        float* mine = part + ((int64_t)tile * ksplit + ks) * NP * 256 + lane * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            __hip_atomic_store(mine + i, g[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (DUAL) __hip_atomic_store(mine + 256 + i, up[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);                         // vmcnt(0)
        asm volatile("" ::: "memory");
        unsigned t = 0;
        if (lane == 0) t = __hip_atomic_fetch_add(&tickets[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        t = __shfl(t, 0, 64);
        if (t != (unsigned)(ksplit - 1)) return;
        asm volatile("" ::: "memory");                              // the partials are read after the ticket is known
        // every ticket of this launch has been drawn: leave the counter at zero for the next one
        if (lane == 0) __hip_atomic_store(&tickets[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int i = 0; i < 4; ++i) g[i] = up[i] = 0.f;
        for (int q = 0; q < ksplit; ++q) {
            const float* src = part + ((int64_t)tile * ksplit + q) * NP * 256 + lane * 4;
#pragma unroll
            for (int i = 0; i < 4; ++i) {                           // device-scope loads: the partials come from other CUs
                g[i] += __hip_atomic_load(src + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (DUAL) up[i] += __hip_atomic_load(src + 256 + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    const int n = tile * 16 + c;
    if (n >= N) return;
    const float bv = bias ? SkinnyT<T>::ld(bias, n) : 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = 4 * kg + i;                // D: lane holds rows 4 kg .. 4 kg + 3 of column c
        if (m >= M) continue;
        // out_f32: the f32 accumulator (plus an f32 residual) is stored as it is
        const float r = residual ? (out_f32 ? reinterpret_cast<const float*>(residual)[(int64_t)m * N + n]
                                            : SkinnyT<T>::ld(residual, (int64_t)m * N + n)) : 0.f;
        const float o = skinny_finish(g[i], up[i], DUAL, act, bv, residual != nullptr, r);
        if (out_f32) reinterpret_cast<float*>(y)[(int64_t)m * N + n] = o;
        else SkinnyT<T>::st(y, (int64_t)m * N + n, o);
    }
}

// Qs[tile][S][lane = 16 kg + c][16 bytes]: byte i = code row (RPW S + RPL kg + i) of column 16 tile + c, xor flip.  int8:
// code rows are k, RPL = 16 rows per lane, flip 0x80.  int4: a code row is a packed byte of two k, RPL = 16 rows (32 k)
// per lane, flip 0x88.  Rows and columns outside the matrix hold the biased zero.
__global__ __launch_bounds__(256) void skinny_pack_codes_kernel(const uint8_t* __restrict__ q, uint8_t* __restrict__ out, int64_t rows,
                                                                int64_t N, int64_t S, int64_t ntiles, uint32_t flip) {
    const int64_t total = ntiles * S * 64;
    for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < total; g += (int64_t)gridDim.x * blockDim.x) {
        const int lane = (int)(g & 63), c = lane & 15, kg = lane >> 4;
        const int64_t sidx = (g >> 6) % S, tile = (g >> 6) / S;
        const int64_t col = tile * 16 + c, r0 = sidx * 64 + kg * 16;
        uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int64_t r = r0 + i;
            const uint32_t b = (col < N && r < rows) ? ((uint32_t)q[r * N + col] ^ flip) : flip;
            w[i >> 2] |= b << (8 * (i & 3));
        }
        *reinterpret_cast<uint4*>(out + g * 16) = make_uint4(w[0], w[1], w[2], w[3]);
    }
}

__device__ __forceinline__ bf16x8_s codes_to_bf16(float f0, float f1, float f2, float f3, float f4, float f5, float f6, float f7) {
    typedef float f32x2_s __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_s __attribute__((ext_vector_type(2)));
    bf16x8_s r;
    const float f[8] = {f0, f1, f2, f3, f4, f5, f6, f7};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f32x2_s p;
        p.x = f[2 * i]; p.y = f[2 * i + 1];
        const bf16x2_s h = __builtin_convertvector(p, bf16x2_s);   // exact: integers below 256
        r[2 * i] = h.x; r[2 * i + 1] = h.y;
    }
    return r;
}
// 8 consecutive int8 codes (two dwords, biased by 128) as the B operand
__device__ __forceinline__ bf16x8_s bytes_to_bf16(uint32_t a, uint32_t b) {
    return codes_to_bf16((float)(a & 0xFFu), (float)((a >> 8) & 0xFFu), (float)((a >> 16) & 0xFFu), (float)(a >> 24),
                         (float)(b & 0xFFu), (float)((b >> 8) & 0xFFu), (float)((b >> 16) & 0xFFu), (float)(b >> 24));
}
// 8 consecutive int4 codes (one dword of packed bytes: k = 2 j in the low nibble of byte j, biased by 8)
__device__ __forceinline__ bf16x8_s nibbles_to_bf16(uint32_t w) {
    const uint32_t lo = w & 0x0F0F0F0Fu, hi = (w >> 4) & 0x0F0F0F0Fu;
    return codes_to_bf16((float)(lo & 0xFFu), (float)(hi & 0xFFu), (float)((lo >> 8) & 0xFFu), (float)((hi >> 8) & 0xFFu),
                         (float)((lo >> 16) & 0xFFu), (float)((hi >> 16) & 0xFFu), (float)(lo >> 24), (float)(hi >> 24));
}

// QF 1: int8, per-column scales [N]; QF 2: int4 in groups of 128, scales [K/128, N].  A word covers KPW = 64 / 128 k.
template <int QF, bool DUAL>
__global__ __launch_bounds__(256) void skinny_gemm_quant_kernel(const bf16_t* __restrict__ x, const uint8_t* __restrict__ qs,
                                                                const uint8_t* __restrict__ qs2, const bf16_t* __restrict__ sc,
                                                                const bf16_t* __restrict__ sc2, const bf16_t* __restrict__ bias,
                                                                const bf16_t* __restrict__ residual, bf16_t* __restrict__ y, int M, int K,
                                                                int N, int act, float* __restrict__ part, unsigned* __restrict__ tickets,
                                                                int out_f32) {
    constexpr int U = 4;                         // words per wave and round, all requested before the first is used
    constexpr int KPW = QF == 1 ? 64 : 128;      // k per word
    constexpr int SPW = KPW / 32;                // MFMA steps per word
    constexpr int NP = DUAL ? 2 : 1;
    constexpr float BIAS = QF == 1 ? 128.0f : 8.0f;
    __shared__ float red[4][NP][64][4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int c = lane & 15, kg = lane >> 4;
    const int tile = blockIdx.x;
    const int ksplit = gridDim.y, ks = blockIdx.y;
    const int nwords = K / KPW;
    const int s_begin = (int)((int64_t)nwords * ks / ksplit), s_end = (int)((int64_t)nwords * (ks + 1) / ksplit);
    const u32x4_s* bsrc = reinterpret_cast<const u32x4_s*>(qs) + (int64_t)tile * nwords * 64 + lane;
    const u32x4_s* bsrc2 = DUAL ? reinterpret_cast<const u32x4_s*>(qs2) + (int64_t)tile * nwords * 64 + lane : nullptr;
    const int arow = c < M ? c : M - 1;
    const bf16_t* arowp = x + (int64_t)arow * K + (KPW / 4) * kg;   // the lane's KPW / 4 consecutive k of a word
    const int ncol = tile * 16 + c < N ? tile * 16 + c : N - 1;     // scale column of this lane's outputs (clamped: never stored)
    bf16x8_s ones;
#pragma unroll
    for (int e = 0; e < 8; ++e) ones[e] = (__bf16)1.0f;

    f32x4_s tot = {0.f, 0.f, 0.f, 0.f}, tot2 = {0.f, 0.f, 0.f, 0.f}, xsum = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = s_begin + wave; s0 < s_end; s0 += 4 * U) {
        u32x4_s b[U], b2[DUAL ? U : 1], a[U][SPW];
        float gs[U], gs2[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int s = s0 + 4 * u < s_end ? s0 + 4 * u : s0;   // a word past the end repeats the first and is skipped below
            b[u] = bsrc[(int64_t)s * 64];
            if (DUAL) b2[u] = bsrc2[(int64_t)s * 64];
#pragma unroll
            for (int t = 0; t < SPW; ++t) a[u][t] = *reinterpret_cast<const u32x4_s*>(arowp + (int64_t)s * KPW + 8 * t);
            if (QF == 2) {
                gs[u] = bf16_to_f32(sc[(int64_t)s * N + ncol]);
                if (DUAL) gs2[u] = bf16_to_f32(sc2[(int64_t)s * N + ncol]);
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (s0 + 4 * u < s_end) {
                f32x4_s acc = {0.f, 0.f, 0.f, 0.f}, acc2 = {0.f, 0.f, 0.f, 0.f}, xs = {0.f, 0.f, 0.f, 0.f};
                const uint32_t bw[4] = {b[u].x, b[u].y, b[u].z, b[u].w};
                const uint32_t bw2[4] = {DUAL ? b2[DUAL ? u : 0].x : 0u, DUAL ? b2[DUAL ? u : 0].y : 0u, DUAL ? b2[DUAL ? u : 0].z : 0u,
                                         DUAL ? b2[DUAL ? u : 0].w : 0u};
#pragma unroll
                for (int t = 0; t < SPW; ++t) {
                    const bf16x8_s av = __builtin_bit_cast(bf16x8_s, a[u][t]);
                    const bf16x8_s bv = QF == 1 ? bytes_to_bf16(bw[2 * t], bw[2 * t + 1]) : nibbles_to_bf16(bw[t]);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, bv, acc, 0, 0, 0);
                    if (DUAL) {
                        const bf16x8_s bv2 = QF == 1 ? bytes_to_bf16(bw2[2 * t], bw2[2 * t + 1]) : nibbles_to_bf16(bw2[t]);
                        acc2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, bv2, acc2, 0, 0, 0);
                    }
                    xs = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, ones, xs, 0, 0, 0);   // sum_k x[row, k] in every column
                }
                if (QF == 1) {
                    tot += acc; xsum += xs;
                    if (DUAL) tot2 += acc2;
                } else {   // one scale group: take the bias out, scale, add
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        tot[i] += gs[u] * (acc[i] - BIAS * xs[i]);
                        if (DUAL) tot2[i] += gs2[u] * (acc2[i] - BIAS * xs[i]);
                    }
                }
            }
        }
    }
    if (QF == 1) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            tot[i] -= BIAS * xsum[i];
            if (DUAL) tot2[i] -= BIAS * xsum[i];
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        red[wave][0][lane][i] = tot[i];
        if (DUAL) red[wave][DUAL ? 1 : 0][lane][i] = tot2[i];
    }
    __syncthreads();
    if (wave != 0) return;
    float g[4], up[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        g[i] = up[i] = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            g[i] += red[w][0][lane][i];
            if (DUAL) up[i] += red[w][DUAL ? 1 : 0][lane][i];
        }
    }
    if (ksplit > 1) {   // as in skinny_gemm_kernel
        float* mine = part + ((int64_t)tile * ksplit + ks) * NP * 256 + lane * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            __hip_atomic_store(mine + i, g[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (DUAL) __hip_atomic_store(mine + 256 + i, up[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);                         // vmcnt(0)
        asm volatile("" ::: "memory");
        unsigned t = 0;
        if (lane == 0) t = __hip_atomic_fetch_add(&tickets[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        t = __shfl(t, 0, 64);
        if (t != (unsigned)(ksplit - 1)) return;
        asm volatile("" ::: "memory");
        if (lane == 0) __hip_atomic_store(&tickets[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int i = 0; i < 4; ++i) g[i] = up[i] = 0.f;
        for (int q = 0; q < ksplit; ++q) {
            const float* src = part + ((int64_t)tile * ksplit + q) * NP * 256 + lane * 4;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                g[i] += __hip_atomic_load(src + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (DUAL) up[i] += __hip_atomic_load(src + 256 + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    const int n = tile * 16 + c;
    if (n >= N) return;
    const float bv = bias ? bf16_to_f32(bias[n]) : 0.f;
    const float s1 = QF == 1 ? bf16_to_f32(sc[n]) : 1.0f;
    const float s2 = QF == 1 && DUAL ? bf16_to_f32(sc2[n]) : 1.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = 4 * kg + i;
        if (m >= M) continue;
        const float r = residual ? (out_f32 ? reinterpret_cast<const float*>(residual)[(int64_t)m * N + n]
                                            : bf16_to_f32(residual[(int64_t)m * N + n])) : 0.f;
        const float o = skinny_finish(g[i] * s1, up[i] * s2, DUAL, act, bv, residual != nullptr, r);
        if (out_f32) reinterpret_cast<float*>(y)[(int64_t)m * N + n] = o;
        else y[(int64_t)m * N + n] = f32_to_bf16(o);
    }
}

}  // namespace

bool skinny_gemm_supported(int dtype, int64_t m, int64_t k, int64_t n) {
    if (dtype != 0 && dtype != 2) return false;
    const int64_t kstep = dtype == 0 ? 16 : 32;
    return m >= 2 && m <= 16 && k >= kstep && k % kstep == 0 && n >= 1 && k < (1ll << 31) && n < (1ll << 31) - 16;
}
size_t skinny_weight_bytes(int dtype, int64_t k, int64_t n) {
    const int64_t kpc = dtype == 0 ? 4 : 8;
    return (size_t)(cdiv_s(n, 16) * cdiv_s(k, kpc) * 16) * 16;
}
void skinny_pack_weights(hipStream_t s, int dtype, const void* w, void* out, int64_t k, int64_t n) {
    const int64_t ntiles = cdiv_s(n, 16), kb = cdiv_s(k, dtype == 0 ? 4 : 8), total = ntiles * kb * 16;
    if (total <= 0) return;
    const unsigned g = (unsigned)(cdiv_s(total, 256) > 65536 ? 65536 : cdiv_s(total, 256));
    if (dtype == 0) skinny_pack_kernel<float><<<g, 256, 0, s>>>((const float*)w, (float*)out, k, n, kb, ntiles);
    else skinny_pack_kernel<bf16_t><<<g, 256, 0, s>>>((const bf16_t*)w, (bf16_t*)out, k, n, kb, ntiles);
}
// Workgroups per tile: doubled while the launch has fewer than two workgroups per CU and each split keeps at least 16
// steps of 32 k (measured on Ministral-3B shapes at 8 rows: 192 tiles x 4 takes 13.8 us where 192 x 1 took 18.7; at
// 576 tiles a split no longer pays).
int skinny_ksplit(int64_t k, int64_t n) {
    const int64_t tiles = cdiv_s(n, 16);
    if (tiles > (int64_t)kSkinnyTickets) return 1;
    int ks = 1;
    while (ks < 8 && tiles * ks < 512 && k / 32 / (ks * 2) >= 16) ks *= 2;
    return ks;
}
size_t skinny_workspace_bytes(int64_t k, int64_t n, bool dual) {
    const int ks = skinny_ksplit(k, n);
    return ks > 1 ? (size_t)cdiv_s(n, 16) * ks * (dual ? 2 : 1) * 256 * sizeof(float) : 0;
}
bool skinny_quant_supported(int dtype, int64_t m, int64_t k, int64_t n, int qf) {
    if ((qf != 1 && qf != 2) || dtype != 2) return false;
    return skinny_gemm_supported(dtype, m, k, n) && k % (qf == 1 ? 64 : 128) == 0;
}
size_t skinny_codes_bytes(int64_t k, int64_t n, int qf) { return (size_t)(cdiv_s(n, 16) * (k / (qf == 1 ? 64 : 128)) * 64 * 16); }
void skinny_pack_codes(hipStream_t s, const void* codes, void* out, int64_t k, int64_t n, int qf) {
    const int64_t ntiles = cdiv_s(n, 16), words = k / (qf == 1 ? 64 : 128), total = ntiles * words * 64;
    if (total <= 0) return;
    const unsigned g = (unsigned)(cdiv_s(total, 256) > 65536 ? 65536 : cdiv_s(total, 256));
    // int8: one code row per k; int4: one packed byte per two k
    skinny_pack_codes_kernel<<<g, 256, 0, s>>>((const uint8_t*)codes, (uint8_t*)out, qf == 1 ? k : k / 2, n, words, ntiles,
                                               qf == 1 ? 0x80u : 0x88u);
}

void skinny_gemm(hipStream_t s, const SkinnyLinearArgs& a) {
    if (a.quant) {
        int ks = skinny_ksplit(a.k / (a.quant == 1 ? 2 : 4), a.n);   // half / a quarter of the bytes per k
        if (!a.part || !a.tickets || a.part_bytes < (size_t)cdiv_s(a.n, 16) * ks * (a.ws2 ? 2 : 1) * 256 * sizeof(float)) ks = 1;
        const dim3 grid((unsigned)cdiv_s(a.n, 16), (unsigned)ks);
#define GPTRS_LAUNCH(QF, DUAL)                                                                                              \
        skinny_gemm_quant_kernel<QF, DUAL><<<grid, 256, 0, s>>>((const bf16_t*)a.x, (const uint8_t*)a.ws, (const uint8_t*)a.ws2,  \
            (const bf16_t*)a.scale, (const bf16_t*)a.scale2, (const bf16_t*)a.bias, (const bf16_t*)a.residual, (bf16_t*)a.y,   \
            (int)a.m, (int)a.k, (int)a.n, a.act, (float*)a.part, a.tickets, a.out_f32)
        if (a.quant == 1) { if (a.ws2) GPTRS_LAUNCH(1, true); else GPTRS_LAUNCH(1, false); }
        else { if (a.ws2) GPTRS_LAUNCH(2, true); else GPTRS_LAUNCH(2, false); }
#undef GPTRS_LAUNCH
        return;
    }
    int ks = skinny_ksplit(a.k, a.n);
    if (!a.part || !a.tickets || a.part_bytes < skinny_workspace_bytes(a.k, a.n, a.ws2 != nullptr)) ks = 1;
    const dim3 grid((unsigned)cdiv_s(a.n, 16), (unsigned)ks);
#define GPTRS_LAUNCH(T, DUAL)                                                                                               \
    skinny_gemm_kernel<T, DUAL><<<grid, 256, 0, s>>>((const T*)a.x, (const T*)a.ws, (const T*)a.ws2, (const T*)a.bias,          \
        (const T*)a.residual, (T*)a.y, (int)a.m, (int)a.k, (int)a.n, a.act, (float*)a.part, a.tickets, a.dtype == 2 ? a.out_f32 : 0)
    if (a.dtype == 0) { if (a.ws2) GPTRS_LAUNCH(float, true); else GPTRS_LAUNCH(float, false); }
    else { if (a.ws2) GPTRS_LAUNCH(bf16_t, true); else GPTRS_LAUNCH(bf16_t, false); }
#undef GPTRS_LAUNCH
}

}  // namespace k
}  // namespace gptrs
