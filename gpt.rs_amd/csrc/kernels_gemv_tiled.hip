// Decode GEMV over a column-tiled copy of the weights.
//
// The reference stores a linear layer's weight as W[in,out] row-major
// (crates/gpt-rs/src/nn/layers/linear.rs:50-71).  For y[M<=16, N] = x . W the backend keeps, per
// weight tensor, a derived layout cached on the device (the role of the reference's derived
// parameters, crates/gpt-rs/src/backend/passes/param_only_fold_to_param.rs:83-147):
//
//     Wt[tile][k][v],  tile = column / VEC,  v = column % VEC,  VEC = 16 bytes / sizeof(T)
//
// i.e. each tile of VEC output columns is ONE contiguous stream of K 16-byte words.  A block owns
// TP tiles for the whole of K, so there is no split-K, no partial sums and no second kernel: lane t
// reads words t, t+256, ... of each of its streams (consecutive lanes -> consecutive 16-byte
// words), multiplies by x[k] staged in LDS and keeps VEC accumulators per tile and row.  The row
// statistic of a preceding RMSNorm costs nothing extra, because every block reads all of x anyway:
// with NORM the kernel computes sum(x^2) itself and scales x while staging it.
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
template <typename T> __device__ __forceinline__ float round_to(float v);
template <> __device__ __forceinline__ float round_to<float>(float v) { return v; }
template <> __device__ __forceinline__ float round_to<bf16_t>(float v) { return bf16_to_f32(f32_to_bf16(v)); }

template <typename T> struct Word;
template <> struct Word<float> {
    static constexpr int VEC = 4;
    static __device__ __forceinline__ void unpack(const uint4& w, float (&o)[4]) {
        o[0] = __uint_as_float(w.x); o[1] = __uint_as_float(w.y); o[2] = __uint_as_float(w.z); o[3] = __uint_as_float(w.w);
    }
};
template <> struct Word<bf16_t> {
    static constexpr int VEC = 8;
    static __device__ __forceinline__ void unpack(const uint4& w, float (&o)[8]) {
        o[0] = bf16lo(w.x); o[1] = bf16hi(w.x); o[2] = bf16lo(w.y); o[3] = bf16hi(w.y);
        o[4] = bf16lo(w.z); o[5] = bf16hi(w.z); o[6] = bf16lo(w.w); o[7] = bf16hi(w.w);
    }
};

// ------------------------------------------------------------------------------ layout transform
template <typename T>
__global__ void tile_weights_kernel(const T* __restrict__ w, T* __restrict__ wt, int64_t K, int64_t N, int64_t ntiles) {
    constexpr int VEC = Word<T>::VEC;
    const int64_t npad = ntiles * VEC, total = K * npad;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t kk = idx / npad, col = idx % npad;
        const T v = col < N ? w[kk * N + col] : T(0);
        wt[((col / VEC) * K + kk) * VEC + (col % VEC)] = v;
    }
}
size_t tiled_weight_bytes(int dtype, int64_t k, int64_t n) {
    const int64_t vec = dtype == 0 ? 4 : 8;
    return (size_t)(cdiv(n, vec) * k * vec) * (dtype == 0 ? 4 : 2);
}
void tile_weights(hipStream_t s, int dtype, const void* w, void* wt, int64_t k, int64_t n) {
    const int64_t vec = dtype == 0 ? 4 : 8, ntiles = cdiv(n, vec), total = k * ntiles * vec;
    if (total <= 0) return;
    const unsigned g = (unsigned)(cdiv(total, 256) > 65536 ? 65536 : cdiv(total, 256));
    if (dtype == 0) tile_weights_kernel<float><<<g, 256, 0, s>>>((const float*)w, (float*)wt, k, n, ntiles);
    else tile_weights_kernel<bf16_t><<<g, 256, 0, s>>>((const bf16_t*)w, (bf16_t*)wt, k, n, ntiles);
}

// ------------------------------------------------------------------------------ GEMV
constexpr int kXsBytes = 32768;  // LDS bytes for the staged activations

__device__ __forceinline__ float tiled_finish(float v, float v2, bool dual, int act, float bias, bool has_res, float res) {
    if (dual) v = (v / (1.0f + expf(v * -1.0f))) * v2;              // activation.rs:141-162
    v += bias;                                                      // tensor_ops.rs:42-56
    if (act == 1) v = (v * 0.5f) * (erff(v / 1.41421354f) + 1.0f);  // activation.rs:96-113
    if (has_res) v += res;
    return v;
}

template <typename T, int MT, int TP, int U, bool DUAL, bool NORM>
__global__ __launch_bounds__(256) void gemv_tiled_kernel(const T* __restrict__ x, const T* __restrict__ wt,
                                                         const T* __restrict__ wt2, const T* __restrict__ gamma,
                                                         const T* __restrict__ beta,
                                                         const T* __restrict__ bias, const T* __restrict__ residual,
                                                         T* __restrict__ y, int M, int64_t K, int64_t N, int64_t ntiles,
                                                         float inv_n, float eps, int act, int out_f32, int x_f32) {
    constexpr int VEC = Word<T>::VEC;
    constexpr int KT = kXsBytes / (int)sizeof(T) / MT;   // rows of x staged at a time (kept as T)
    constexpr int PLANE = TP * MT * VEC;                 // outputs per block (per weight stream set)
    constexpr int NOUT = PLANE * (DUAL ? 2 : 1);
    __shared__ T xs[MT][KT];
    __shared__ float red[4][NOUT];
    __shared__ float s_scale[MT];
    __shared__ float s_mean[MT];
    __shared__ float s_tmp[16];
    const int t = threadIdx.x;
    const int64_t tile0 = (int64_t)blockIdx.x * TP;

    const uint4* streams[TP];
    const uint4* streams2[DUAL ? TP : 1];
#pragma unroll
    for (int p = 0; p < TP; ++p) {
        // a block's last tiles may fall past the end: point them at the last valid tile, skip the store
        const int64_t tile = tile0 + p < ntiles ? tile0 + p : ntiles - 1;
        streams[p] = reinterpret_cast<const uint4*>(wt) + tile * K;
        if (DUAL) streams2[p] = reinterpret_cast<const uint4*>(wt2) + tile * K;
    }

    // The first batch of weight words is requested before anything else, so the staging of x (and
    // the row statistic of a fused RMSNorm) overlaps their flight instead of preceding it.
    uint4 w[U][TP];
    uint4 w2[DUAL ? U : 1][TP];
    const int64_t kt_first = K < KT ? K : KT;
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int64_t r = (int64_t)t + (int64_t)u * 256;
        const int64_t rc = r < kt_first ? r : 0;  // dead slots re-read word 0, multiplied by zero below
#pragma unroll
        for (int p = 0; p < TP; ++p) {
            w[u][p] = streams[p][rc];
            if (DUAL) w2[u][p] = streams2[p][rc];
        }
    }

    // RMSNorm prologue (normalization.rs:183-217): inv_rms = rsqrt(sum(x^2)*(1/N) + eps) per row.
    // When the whole row fits the staging buffer the same pass also stages x (raw); the scaling
    // pass below then touches only LDS and gamma.
    // LayerNorm (beta given; normalization.rs:123-174): mean first, then the variance of the centred values, as the
    // stand-alone kernel takes them.
    // x_f32 (RMSNorm only): x and gamma are f32; the staged row is their f32 norm rounded to T once
    const float* xf = reinterpret_cast<const float*>(x);
    const float* gf = reinterpret_cast<const float*>(gamma);
    const bool one_chunk = K <= KT && !x_f32;
    if (NORM) {
        for (int m = 0; m < M; ++m) {
            float q = 0.f, mean = 0.f;
            if (beta) {
                float sm = 0.f;
                for (int64_t kk = t; kk < K; kk += 256) sm += ldf(x, (int64_t)m * K + kk);
                mean = block_sum(sm, s_tmp) * inv_n;
            }
            for (int64_t kk = t; kk < K; kk += 256) {
                if (x_f32) { const float v = xf[(int64_t)m * K + kk]; q += v * v; continue; }
                const T raw = x[(int64_t)m * K + kk];
                const float v = ldf(&raw, 0) - mean;
                if (one_chunk) xs[m][kk] = raw;
                q += v * v;
            }
            const float tot = block_sum(q, s_tmp);
            if (t == 0) { s_scale[m] = 1.0f / sqrtf(tot * inv_n + eps); s_mean[m] = mean; }
        }
        __syncthreads();
    }

    float acc[TP][MT][VEC];
    float acc2[DUAL ? TP : 1][MT][VEC];
#pragma unroll
    for (int p = 0; p < TP; ++p)
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int v = 0; v < VEC; ++v) { acc[p][m][v] = 0.f; if (DUAL) acc2[p][m][v] = 0.f; }

    for (int64_t k0 = 0; k0 < K; k0 += KT) {
        const int64_t kt = K - k0 < KT ? K - k0 : KT;
        __syncthreads();
        // only the live part of the staging buffer is written: rows m >= M feed accumulators that
        // are never stored, slots past kt are never read
        for (int m = 0; m < M; ++m)
            for (int64_t kk = t; kk < kt; kk += 256) {
                // each thread re-reads only the slots it wrote itself in the prologue
                float v = (NORM && x_f32) ? xf[(int64_t)m * K + k0 + kk]
                                          : ((NORM && one_chunk) ? ldf(&xs[m][0], kk) : ldf(x, (int64_t)m * K + k0 + kk));
                // the value the stand-alone norm kernel would have stored: (x*inv_rms)*gamma, rounded to T
                if (NORM) {
                    v = ((v - s_mean[m]) * s_scale[m]) * (x_f32 ? gf[k0 + kk] : ldf(gamma, k0 + kk));
                    if (beta) v += ldf(beta, k0 + kk);
                }
                stf(&xs[m][0], kk, v);
            }
        __syncthreads();
        for (int64_t r0 = t; r0 < kt; r0 += 256 * U) {
            if (k0 != 0 || r0 != t) {  // the very first batch is already in flight
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int64_t r = r0 + (int64_t)u * 256;
                    const int64_t rc = r < kt ? r : 0;
#pragma unroll
                    for (int p = 0; p < TP; ++p) {
                        w[u][p] = streams[p][k0 + rc];
                        if (DUAL) w2[u][p] = streams2[p][k0 + rc];
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int64_t r = r0 + (int64_t)u * 256;
                const bool live = r < kt;
                const int rr = live ? (int)r : 0;
                float xv[MT];
#pragma unroll
                for (int m = 0; m < MT; ++m) xv[m] = live ? ldf(&xs[m][0], rr) : 0.f;
#pragma unroll
                for (int p = 0; p < TP; ++p) {
                    float wf[VEC], wf2[VEC];
                    Word<T>::unpack(w[u][p], wf);
                    if (DUAL) Word<T>::unpack(w2[u][p], wf2);
#pragma unroll
                    for (int m = 0; m < MT; ++m)
#pragma unroll
                        for (int v = 0; v < VEC; ++v) {
                            acc[p][m][v] = __builtin_fmaf(xv[m], wf[v], acc[p][m][v]);
                            if (DUAL) acc2[p][m][v] = __builtin_fmaf(xv[m], wf2[v], acc2[p][m][v]);
                        }
                }
            }
        }
    }

    // 256 partial sums per output -> one: xor-shuffle inside each wave, then four waves through LDS
    const int lane = t & 63, wave = t >> 6;
#pragma unroll
    for (int p = 0; p < TP; ++p)
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
                float a = wave_sum(acc[p][m][v]);
                if (lane == 0) red[wave][(p * MT + m) * VEC + v] = a;
                if (DUAL) {
                    float b = wave_sum(acc2[p][m][v]);
                    if (lane == 0) red[wave][PLANE + (p * MT + m) * VEC + v] = b;
                }
            }
    __syncthreads();
    for (int o = t; o < PLANE; o += 256) {
        const int v = o % VEC, m = (o / VEC) % MT, p = o / (VEC * MT);
        const int64_t col = (tile0 + p) * VEC + v;
        if (m >= M || tile0 + p >= ntiles || col >= N) continue;
        const float tot = red[0][o] + red[1][o] + red[2][o] + red[3][o];
        const float tot2 = DUAL ? red[0][PLANE + o] + red[1][PLANE + o] + red[2][PLANE + o] + red[3][PLANE + o] : 0.f;
        const float b = bias ? ldf(bias, col) : 0.f;
        // out_f32: the f32 accumulator (plus an f32 residual) is stored as it is
        const float r = residual ? (out_f32 ? reinterpret_cast<const float*>(residual)[(int64_t)m * N + col]
                                            : ldf(residual, (int64_t)m * N + col)) : 0.f;
        const float res = tiled_finish(tot, tot2, DUAL, act, b, residual != nullptr, r);
        if (out_f32) reinterpret_cast<float*>(y)[(int64_t)m * N + col] = res;
        else stf(y, (int64_t)m * N + col, res);
    }
}

bool gemv_tiled_supported(int dtype, int64_t m, int64_t k, int64_t n) {
    return (dtype == 0 || dtype == 2) && m >= 1 && m <= 16 && k >= 1 && n >= 1;
}

template <typename T, int MT, int TP, int U>
static void launch_tiled(hipStream_t s, const TiledLinearArgs& a) {
    constexpr int VEC = Word<T>::VEC;
    const int64_t ntiles = cdiv(a.n, VEC);
    const unsigned grid = (unsigned)cdiv(ntiles, TP);
#define GPTRS_GT(DUAL, NORM)                                                                                          \
    gemv_tiled_kernel<T, MT, TP, U, DUAL, NORM><<<grid, 256, 0, s>>>((const T*)a.x, (const T*)a.wt, (const T*)a.wt2,         \
        (const T*)a.gamma, (const T*)a.beta, (const T*)a.bias, (const T*)a.residual, (T*)a.y, (int)a.m, a.k, a.n, ntiles, a.inv_n, a.eps, a.act, \
        sizeof(T) == 2 ? a.out_f32 : 0, sizeof(T) == 2 ? a.x_f32 : 0)
    if (a.wt2) { if (a.gamma) GPTRS_GT(true, true); else GPTRS_GT(true, false); }
    else { if (a.gamma) GPTRS_GT(false, true); else GPTRS_GT(false, false); }
#undef GPTRS_GT
}
template <typename T>
static void gemv_tiled_t(hipStream_t s, const TiledLinearArgs& a) {
    constexpr int VEC = Word<T>::VEC;
    const int64_t ntiles = cdiv(a.n, VEC);
    // several tiles per block once there are more tiles than ~8 blocks per CU can hold at once;
    // more words in flight per lane when there are few blocks (small N) to cover the latency
    const bool many = ntiles > 4096;
    const bool few = ntiles <= 512;
    if (a.m <= 1) {
        if (many) launch_tiled<T, 1, 4, 2>(s, a);
        else if (few) launch_tiled<T, 1, 1, 8>(s, a);
        else launch_tiled<T, 1, 1, 4>(s, a);
    } else if (a.m <= 2) {
        if (many) launch_tiled<T, 2, 2, 2>(s, a); else launch_tiled<T, 2, 1, 4>(s, a);
    } else if (a.m <= 4) {
        if (many) launch_tiled<T, 4, 2, 2>(s, a); else launch_tiled<T, 4, 1, 4>(s, a);
    } else if (a.m <= 8) {
        launch_tiled<T, 8, 1, 2>(s, a);
    } else {
        launch_tiled<T, 16, 1, 2>(s, a);
    }
}
void gemv_tiled(hipStream_t s, const TiledLinearArgs& a) {
    if (a.m <= 0 || a.n <= 0) return;
    if (a.dtype == 0) gemv_tiled_t<float>(s, a);
    else gemv_tiled_t<bf16_t>(s, a);
}

// The inverse of the decode chain's bf16 weight copy (kernels_chain.hip: 4-column tiles, word j of a column holds rows
// 2j and 2j + 1; a pair of matrices interleaves its columns gate, up, gate, up inside a tile): the row-major [K, N]
// matrix back, exactly -- the copy is a permutation plus zero padding.  A matrix whose packed copy exists need not stay
// resident in its row-major form; this brings it back when some other kernel family asks for it.
__global__ void chain_unpack_kernel(const uint32_t* __restrict__ packed, bf16_t* __restrict__ w, bf16_t* __restrict__ w2,
                                    int64_t K, int64_t N, int64_t Kw, int dual) {
    const int64_t total = Kw * N;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t col = idx % N, j = idx / N;
        if (2 * j >= K) continue;
        const bool two = 2 * j + 1 < K;
        if (!dual) {
            const uint32_t v = packed[((col >> 2) * Kw + j) * 4 + (col & 3)];
            w[(2 * j) * N + col] = (bf16_t)(v & 0xFFFFu);
            if (two) w[(2 * j + 1) * N + col] = (bf16_t)(v >> 16);
        } else {
            const int64_t base = ((col >> 1) * Kw + j) * 4 + ((col & 1) << 1);
            if (w) {
                const uint32_t v = packed[base];
                w[(2 * j) * N + col] = (bf16_t)(v & 0xFFFFu);
                if (two) w[(2 * j + 1) * N + col] = (bf16_t)(v >> 16);
            }
            if (w2) {
                const uint32_t v = packed[base + 1];
                w2[(2 * j) * N + col] = (bf16_t)(v & 0xFFFFu);
                if (two) w2[(2 * j + 1) * N + col] = (bf16_t)(v >> 16);
            }
        }
    }
}

void chain_unpack_weights(hipStream_t s, const void* packed, void* w, void* w2, int64_t k, int64_t n, bool dual) {
    const int64_t ntiles = ((dual ? 2 * n : n) + 3) / 4;
    if (ntiles <= 0 || k <= 0 || (!w && !w2)) return;
    const int64_t kw = (int64_t)(chain_weight_bytes(k, n, dual, kChainW16) / (size_t)(16 * ntiles));   // words per column
    const int64_t total = kw * n;
    const unsigned g = (unsigned)std::min<int64_t>((total + 255) / 256, 65536);
    chain_unpack_kernel<<<g, 256, 0, s>>>((const uint32_t*)packed, (bf16_t*)w, (bf16_t*)w2, k, n, kw, dual ? 1 : 0);
}


}  // namespace k
}  // namespace gptrs
