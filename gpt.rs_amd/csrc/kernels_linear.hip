// Linear layers: y[M,N] = act(x[M,K] . W[K,N] + bias) (+ residual), W row-major [in,out] as the
// reference stores it (crates/gpt-rs/src/nn/layers/linear.rs:50-71).
//
//  * M <= 16  (decode): HBM-bound GEMV.  Lanes run along N so every wave load is a run of
//    contiguous 16-byte words of one weight row; K is split across the 16 row-groups of a block
//    and across blockIdx.y; partial sums meet in LDS, then (split-K) in a scratch buffer that a
//    small second kernel sums in a fixed order, so results are run-to-run identical.
//  * M > 16   (prefill): tiled GEMM (gemm_tiled below; MFMA tiles live in kernels_mfma.hip).
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

// VEC consecutive weights of one row as f32.  VEC*sizeof(T) == 16 uses one 128-bit load.
template <typename T, int VEC> struct RowVec;
template <> struct RowVec<float, 4> {
    static __device__ __forceinline__ void load(const float* p, float (&o)[4]) {
        const float4 v = *reinterpret_cast<const float4*>(p);
        o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
    }
};
template <> struct RowVec<bf16_t, 8> {
    static __device__ __forceinline__ void load(const bf16_t* p, float (&o)[8]) {
        const uint4 v = *reinterpret_cast<const uint4*>(p);
        o[0] = bf16lo(v.x); o[1] = bf16hi(v.x); o[2] = bf16lo(v.y); o[3] = bf16hi(v.y);
        o[4] = bf16lo(v.z); o[5] = bf16hi(v.z); o[6] = bf16lo(v.w); o[7] = bf16hi(v.w);
    }
};
template <typename T> struct RowVec<T, 1> {
    static __device__ __forceinline__ void load(const T* p, float (&o)[1]) { o[0] = ldf(p, 0); }
};

__device__ __forceinline__ float finish(float v, float v2, bool dual, int act, float bias, bool has_res, float res) {
    if (dual) v = (v / (1.0f + expf(v * -1.0f))) * v2;        // activation.rs:141-162
    v += bias;                                                // tensor_ops.rs:42-56
    if (act == 1) v = (v * 0.5f) * (erff(v / 1.41421354f) + 1.0f);  // activation.rs:96-113
    if (has_res) v += res;
    return v;
}

constexpr int kGemvKT = 512;  // rows of x staged in LDS at a time

template <typename T, int VEC, int MT, bool DUAL>
__global__ __launch_bounds__(256) void gemv_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                   const T* __restrict__ w2, const T* __restrict__ bias,
                                                   const T* __restrict__ residual, T* __restrict__ y,
                                                   float* __restrict__ partial, int* __restrict__ counters, int M,
                                                   int64_t K, int64_t N, int64_t kc, int act) {
    constexpr int LN = VEC == 1 ? 64 : 16;  // lanes along N
    constexpr int RG = 256 / LN;            // row groups per block
    constexpr int CT = LN * VEC;            // columns per block
    constexpr int U = MT >= 16 ? 2 : 4;      // rows in flight per thread
    __shared__ float xs[MT][kGemvKT];
    __shared__ float red[RG][CT + 1];

    const int cn = threadIdx.x % LN, rg = threadIdx.x / LN;
    const int64_t col = (int64_t)blockIdx.x * CT + (int64_t)cn * VEC;
    const bool col_ok = col < N;
    const int S = gridDim.y;
    const int64_t k_begin = (int64_t)blockIdx.y * kc;
    const int64_t k_end = k_begin + kc < K ? k_begin + kc : K;

    float acc[MT][VEC];
    float acc2[DUAL ? MT : 1][VEC];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int v = 0; v < VEC; ++v) { acc[m][v] = 0.f; if (DUAL) acc2[m][v] = 0.f; }

    for (int64_t k0 = k_begin; k0 < k_end; k0 += kGemvKT) {
        const int64_t kt = k_end - k0 < kGemvKT ? k_end - k0 : kGemvKT;
        __syncthreads();
        for (int i = threadIdx.x; i < MT * kGemvKT; i += 256) {
            const int m = i / kGemvKT, kk = i % kGemvKT;
            xs[m][kk] = (m < M && kk < kt) ? ldf(x, (int64_t)m * K + k0 + kk) : 0.f;
        }
        __syncthreads();
        if (col_ok) {
            for (int64_t r0 = rg; r0 < kt; r0 += RG * U) {
                float wv[U][VEC];
                float wv2[DUAL ? U : 1][VEC];
                // all U loads are issued before any is consumed; rows past the end re-read the last
                // valid row and are multiplied by zero
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int64_t r = r0 + (int64_t)u * RG;
                    const int64_t rc = r < kt ? r : kt - 1;
                    RowVec<T, VEC>::load(w + (k0 + rc) * N + col, wv[u]);
                    if (DUAL) RowVec<T, VEC>::load(w2 + (k0 + rc) * N + col, wv2[u]);
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int64_t r = r0 + (int64_t)u * RG;
                    const bool live = r < kt;
                    const int rr = live ? (int)r : 0;
#pragma unroll
                    for (int m = 0; m < MT; ++m) {
                        const float xv = live ? xs[m][rr] : 0.f;
#pragma unroll
                        for (int v = 0; v < VEC; ++v) {
                            acc[m][v] = __builtin_fmaf(xv, wv[u][v], acc[m][v]);
                            if (DUAL) acc2[m][v] = __builtin_fmaf(xv, wv2[u][v], acc2[m][v]);
                        }
                    }
                }
            }
        }
    }

    // ---- meet the RG row-groups in LDS, one output row at a time.  The loops over m are fully
    // unrolled (static register indices); rows m >= M leave through a block-uniform branch.
    const int t = threadIdx.x;
    const int64_t ocol = (int64_t)blockIdx.x * CT + t;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        if (m >= M) break;
        float tot = 0.f, tot2 = 0.f;
#pragma unroll
        for (int pass = 0; pass < (DUAL ? 2 : 1); ++pass) {
            __syncthreads();
#pragma unroll
            for (int v = 0; v < VEC; ++v) red[rg][cn * VEC + v] = pass == 0 ? acc[m][v] : acc2[DUAL ? m : 0][v];
            __syncthreads();
            if (t < CT) {
                float sacc = 0.f;
#pragma unroll
                for (int g = 0; g < RG; ++g) sacc += red[g][t];
                if (pass == 0) tot = sacc; else tot2 = sacc;
            }
        }
        if (t < CT && ocol < N) {
            if (S == 1) {
                const float b = bias ? ldf(bias, ocol) : 0.f;
                const float r = residual ? ldf(residual, (int64_t)m * N + ocol) : 0.f;
                stf(y, (int64_t)m * N + ocol, finish(tot, tot2, DUAL, act, b, residual != nullptr, r));
            } else {
                partial[((int64_t)blockIdx.y * M + m) * N + ocol] = tot;
                if (DUAL) partial[((int64_t)(S + blockIdx.y) * M + m) * N + ocol] = tot2;
            }
        }
    }
}

// Split-K epilogue: sums the S slices in a fixed order (run-to-run identical results) and applies
// bias / activation / residual.  A separate launch, because a grid-wide "last block finishes"
// scheme needs device-scope fences, and on this multi-XCD part each such fence writes back and
// invalidates a whole L2: measured ~90 us per GEMV, against ~3 us for this kernel.
template <typename T, bool DUAL>
__global__ void gemv_reduce_kernel(const float* __restrict__ partial, const T* __restrict__ bias,
                                   const T* __restrict__ residual, T* __restrict__ y, int M, int64_t N, int S, int act) {
    const int64_t total = (int64_t)M * N;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t col = idx % N;
        float tot = 0.f, tot2 = 0.f;
#pragma unroll 8
        for (int sidx = 0; sidx < S; ++sidx) {
            tot += partial[(int64_t)sidx * total + idx];
            if (DUAL) tot2 += partial[(int64_t)(S + sidx) * total + idx];
        }
        const float b = bias ? ldf(bias, col) : 0.f;
        const float r = residual ? ldf(residual, idx) : 0.f;
        stf(y, idx, finish(tot, tot2, DUAL, act, b, residual != nullptr, r));
    }
}

// Launch geometry shared by linear() and linear_workspace_bytes().
struct GemvPlan {
    int vec, ct, tiles, splits;
    int64_t kc;
};
constexpr int kMaxCounterTiles = 4096;
static GemvPlan plan_gemv(int dtype, int64_t k, int64_t n, bool aligned) {
    GemvPlan p;
    const int full = dtype == 0 ? 4 : 8;
    p.vec = aligned ? full : 1;
    p.ct = p.vec == 1 ? 64 : 16 * p.vec;
    p.tiles = (int)cdiv(n, p.ct);
    // aim for ~4 blocks on each of the 256 CUs, at least 64 rows of K per block
    int64_t want = cdiv(1024, p.tiles);
    int64_t max_by_k = k / 64 > 0 ? k / 64 : 1;
    int64_t s = want < max_by_k ? want : max_by_k;
    if (s < 1) s = 1;
    if (s > 64) s = 64;
    if (p.tiles > kMaxCounterTiles) s = 1;
    p.kc = cdiv(cdiv(k, s), 16) * 16;
    p.splits = (int)cdiv(k, p.kc);
    return p;
}
static bool gemv_aligned(int dtype, int64_t n, const void* w, const void* w2) {
    const int full = dtype == 0 ? 4 : 8;
    return n % full == 0 && ((uintptr_t)w % 16 == 0) && ((uintptr_t)w2 % 16 == 0);
}

template <typename T, int VEC, int MT>
static void launch_gemv(hipStream_t s, const LinearArgs& a, const GemvPlan& p, float* partial, int* counters) {
    dim3 grid((unsigned)p.tiles, (unsigned)p.splits);
    if (a.w2)
        gemv_kernel<T, VEC, MT, true><<<grid, 256, 0, s>>>((const T*)a.x, (const T*)a.w, (const T*)a.w2, (const T*)a.bias,
            (const T*)a.residual, (T*)a.y, partial, counters, (int)a.m, a.k, a.n, p.kc, a.act);
    else
        gemv_kernel<T, VEC, MT, false><<<grid, 256, 0, s>>>((const T*)a.x, (const T*)a.w, nullptr, (const T*)a.bias,
            (const T*)a.residual, (T*)a.y, partial, counters, (int)a.m, a.k, a.n, p.kc, a.act);
    if (p.splits > 1) {
        const int64_t total = a.m * a.n;
        const unsigned g = (unsigned)(cdiv(total, 256) > 2048 ? 2048 : cdiv(total, 256));
        if (a.w2)
            gemv_reduce_kernel<T, true><<<g, 256, 0, s>>>(partial, (const T*)a.bias, (const T*)a.residual, (T*)a.y, (int)a.m, a.n, p.splits, a.act);
        else
            gemv_reduce_kernel<T, false><<<g, 256, 0, s>>>(partial, (const T*)a.bias, (const T*)a.residual, (T*)a.y, (int)a.m, a.n, p.splits, a.act);
    }
}
template <typename T, int VEC>
static void launch_gemv_m(hipStream_t s, const LinearArgs& a, const GemvPlan& p, float* partial, int* counters) {
    if (a.m <= 1) launch_gemv<T, VEC, 1>(s, a, p, partial, counters);
    else if (a.m <= 2) launch_gemv<T, VEC, 2>(s, a, p, partial, counters);
    else if (a.m <= 4) launch_gemv<T, VEC, 4>(s, a, p, partial, counters);
    else if (a.m <= 8) launch_gemv<T, VEC, 8>(s, a, p, partial, counters);
    else launch_gemv<T, VEC, 16>(s, a, p, partial, counters);
}

// ------------------------------------------------------------------------------ tiled GEMM (M > 16)
// 64x64 output tile, BK = 16, 256 threads, 4x4 outputs per thread, f32 accumulate.
template <typename T>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                         const T* __restrict__ bias, const T* __restrict__ residual,
                                                         T* __restrict__ y, int64_t M, int64_t K, int64_t N, int act) {
    __shared__ float As[16][64 + 4];
    __shared__ float Bs[16][64 + 4];
    const int64_t m0 = (int64_t)blockIdx.y * 64, n0 = (int64_t)blockIdx.x * 64;
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    float acc[4][4] = {};
    for (int64_t k0 = 0; k0 < K; k0 += 16) {
        // A tile: 64 rows x 16 k  (thread -> row = tid/4, 4 consecutive k)
        {
            const int r = threadIdx.x >> 2, kk = (threadIdx.x & 3) * 4;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int64_t m = m0 + r, kx = k0 + kk + j;
                As[kk + j][r] = (m < M && kx < K) ? ldf(x, m * K + kx) : 0.f;
            }
        }
        // B tile: 16 k x 64 n  (thread -> k = tid/16, 4 consecutive n)
        {
            const int kk = threadIdx.x >> 4, c = (threadIdx.x & 15) * 4;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int64_t kx = k0 + kk, n = n0 + c + j;
                Bs[kk][c + j] = (kx < K && n < N) ? ldf(w, kx * N + n) : 0.f;
            }
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) {
            float av[4], bv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { av[i] = As[kk][ty * 4 + i]; bv[i] = Bs[kk][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] += av[i] * bv[j];
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int64_t m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t n = n0 + tx * 4 + j;
            if (n >= N) continue;
            const float b = bias ? ldf(bias, n) : 0.f;
            const float r = residual ? ldf(residual, m * N + n) : 0.f;
            stf(y, m * N + n, finish(acc[i][j], 0.f, false, act, b, residual != nullptr, r));
        }
    }
}

static void gemm_any(hipStream_t s, int dtype, const void* x, const void* w, const void* bias, const void* residual,
                     void* y, int64_t m, int64_t k, int64_t n, int act) {
    dim3 grid((unsigned)cdiv(n, 64), (unsigned)cdiv(m, 64));
    if (dtype == 0)
        gemm_tiled_kernel<float><<<grid, 256, 0, s>>>((const float*)x, (const float*)w, (const float*)bias, (const float*)residual, (float*)y, m, k, n, act);
    else
        gemm_tiled_kernel<bf16_t><<<grid, 256, 0, s>>>((const bf16_t*)x, (const bf16_t*)w, (const bf16_t*)bias, (const bf16_t*)residual, (bf16_t*)y, m, k, n, act);
}

// ------------------------------------------------------------------------------ entry points
size_t linear_workspace_bytes(int dtype, int64_t m, int64_t k, int64_t n, bool dual) {
    if (m <= 16) {
        // split-K partial sums [planes][splits][M][N] f32; bound over both load widths
        size_t best = 0;
        for (int al = 0; al < 2; ++al) {
            const GemvPlan p = plan_gemv(dtype, k, n, al != 0);
            const size_t b = p.splits > 1 ? (size_t)(dual ? 2 : 1) * p.splits * (size_t)m * (size_t)n * sizeof(float) : 0;
            if (b > best) best = b;
        }
        return best;
    }
    const size_t es = dtype == 0 ? 4 : 2;
    return dual ? 2 * (size_t)m * (size_t)n * es : 0;
}

void linear(hipStream_t s, const LinearArgs& a) {
    if (a.m <= 0 || a.n <= 0) return;
    if (a.m <= 16) {
        const GemvPlan p = plan_gemv(a.dtype, a.k, a.n, gemv_aligned(a.dtype, a.n, a.w, a.w2));
        int* counters = a.counters;
        float* partial = (float*)a.ws;
        if (a.dtype == 0) {
            if (p.vec == 4) launch_gemv_m<float, 4>(s, a, p, partial, counters);
            else launch_gemv_m<float, 1>(s, a, p, partial, counters);
        } else {
            if (p.vec == 8) launch_gemv_m<bf16_t, 8>(s, a, p, partial, counters);
            else launch_gemv_m<bf16_t, 1>(s, a, p, partial, counters);
        }
        return;
    }
    if (!a.w2) {
        gemm_any(s, a.dtype, a.x, a.w, a.bias, a.residual, a.y, a.m, a.k, a.n, a.act);
        return;
    }
    // SwiGLU pair at prefill sizes: two GEMMs into scratch, then the gating kernel
    const size_t es = a.dtype == 0 ? 4 : 2;
    void* g = a.ws;
    void* u = (char*)a.ws + (size_t)a.m * a.n * es;
    gemm_any(s, a.dtype, a.x, a.w, nullptr, nullptr, g, a.m, a.k, a.n, 0);
    gemm_any(s, a.dtype, a.x, a.w2, nullptr, nullptr, u, a.m, a.k, a.n, 0);
    swiglu(s, a.dtype, g, u, a.y, a.m * a.n);
}

}  // namespace k
}  // namespace gptrs
