// Fused kernels for the functional sequences of the LM path: row norms, softmax, GELU/SwiGLU,
// packed RoPE.  Each replaces an exact PTIR op sequence emitted by
// crates/gpt-rs/src/ops/functional/*.rs; math is f32 with one rounding to the output dtype.
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

// ------------------------------------------------------------------------------ layer_norm
// normalization.rs:123-174: mean = sum*(1/N); c = x-mean; var = sum(c*c)*(1/N); y = c*rsqrt(var+eps)*g+b
// One block per row; the row stays in registers between the passes (up to 16 values/thread).
template <typename T, int PER>
__global__ void layer_norm_kernel(const T* __restrict__ x, const T* __restrict__ gamma, const T* __restrict__ beta,
                                  T* __restrict__ y, int64_t n, float inv_n, float eps) {
    __shared__ float red[16];
    const T* row = x + (int64_t)blockIdx.x * n;
    T* out = y + (int64_t)blockIdx.x * n;
    float v[PER];
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int64_t i = threadIdx.x + (int64_t)j * blockDim.x;
        v[j] = i < n ? ldf(row, i) : 0.f;
        s += v[j];
    }
    const float mean = block_sum(s, red) * inv_n;
    float q = 0.f;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int64_t i = threadIdx.x + (int64_t)j * blockDim.x;
        const float c = i < n ? v[j] - mean : 0.f;
        v[j] = c;
        q += c * c;
    }
    const float var = block_sum(q, red) * inv_n;
    const float inv_std = 1.0f / sqrtf(var + eps);
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int64_t i = threadIdx.x + (int64_t)j * blockDim.x;
        if (i < n) stf(out, i, (v[j] * inv_std) * ldf(gamma, i) + ldf(beta, i));
    }
}
// rows longer than 16*blockDim: re-read from memory on each pass
template <typename T>
__global__ void layer_norm_long_kernel(const T* __restrict__ x, const T* __restrict__ gamma, const T* __restrict__ beta,
                                       T* __restrict__ y, int64_t n, float inv_n, float eps) {
    __shared__ float red[16];
    const T* row = x + (int64_t)blockIdx.x * n;
    T* out = y + (int64_t)blockIdx.x * n;
    float s = 0.f;
    for (int64_t i = threadIdx.x; i < n; i += blockDim.x) s += ldf(row, i);
    const float mean = block_sum(s, red) * inv_n;
    float q = 0.f;
    for (int64_t i = threadIdx.x; i < n; i += blockDim.x) { const float c = ldf(row, i) - mean; q += c * c; }
    const float inv_std = 1.0f / sqrtf(block_sum(q, red) * inv_n + eps);
    for (int64_t i = threadIdx.x; i < n; i += blockDim.x)
        stf(out, i, ((ldf(row, i) - mean) * inv_std) * ldf(gamma, i) + ldf(beta, i));
}

template <typename T>
static void layer_norm_t(hipStream_t s, const T* x, const T* g, const T* b, T* y, int64_t rows, int64_t n, float inv_n,
                         float eps) {
    const int block = n <= 256 ? 64 : (n <= 1024 ? 256 : 1024);  // decode has ONE row: spread it over many lanes
    const int64_t per = cdiv(n, block);
    const unsigned grid = (unsigned)rows;
    if (per <= 4) layer_norm_kernel<T, 4><<<grid, block, 0, s>>>(x, g, b, y, n, inv_n, eps);
    else if (per <= 16) layer_norm_kernel<T, 16><<<grid, block, 0, s>>>(x, g, b, y, n, inv_n, eps);
    else layer_norm_long_kernel<T><<<grid, 1024, 0, s>>>(x, g, b, y, n, inv_n, eps);
}
void layer_norm(hipStream_t s, int dtype, const void* x, const void* gamma, const void* beta, void* y, int64_t rows,
                int64_t n, float inv_n, float eps) {
    if (rows <= 0 || n <= 0) return;
    if (dtype == 0) layer_norm_t<float>(s, (const float*)x, (const float*)gamma, (const float*)beta, (float*)y, rows, n, inv_n, eps);
    else layer_norm_t<bf16_t>(s, (const bf16_t*)x, (const bf16_t*)gamma, (const bf16_t*)beta, (bf16_t*)y, rows, n, inv_n, eps);
}

// ------------------------------------------------------------------------------ rms_norm
// normalization.rs:183-217: y = (x * rsqrt(sum(x*x)*(1/N) + eps)) * gamma
template <typename T, int PER>
__global__ void rms_norm_kernel(const T* __restrict__ x, const T* __restrict__ gamma, T* __restrict__ y, int64_t n,
                                float inv_n, float eps) {
    __shared__ float red[16];
    const T* row = x + (int64_t)blockIdx.x * n;
    T* out = y + (int64_t)blockIdx.x * n;
    float v[PER];
    float q = 0.f;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int64_t i = threadIdx.x + (int64_t)j * blockDim.x;
        v[j] = i < n ? ldf(row, i) : 0.f;
        q += v[j] * v[j];
    }
    const float inv_rms = 1.0f / sqrtf(block_sum(q, red) * inv_n + eps);
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int64_t i = threadIdx.x + (int64_t)j * blockDim.x;
        if (i < n) stf(out, i, (v[j] * inv_rms) * ldf(gamma, i));
    }
}
template <typename T>
__global__ void rms_norm_long_kernel(const T* __restrict__ x, const T* __restrict__ gamma, T* __restrict__ y, int64_t n,
                                     float inv_n, float eps) {
    __shared__ float red[16];
    const T* row = x + (int64_t)blockIdx.x * n;
    T* out = y + (int64_t)blockIdx.x * n;
    float q = 0.f;
    for (int64_t i = threadIdx.x; i < n; i += blockDim.x) { const float v = ldf(row, i); q += v * v; }
    const float inv_rms = 1.0f / sqrtf(block_sum(q, red) * inv_n + eps);
    for (int64_t i = threadIdx.x; i < n; i += blockDim.x) stf(out, i, (ldf(row, i) * inv_rms) * ldf(gamma, i));
}
// bf16 rows of up to 8192 values whose length is a multiple of 8: one 16-byte load and store per thread (the kernels
// above move 2 bytes per lane and instruction, which at 1024 rows of 3072 took 8.6 us per launch)
typedef uint32_t fused_u32x4_t __attribute__((ext_vector_type(4)));
__global__ void rms_norm_vec_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ gamma, bf16_t* __restrict__ y,
                                    int64_t n, float inv_n, float eps) {
    __shared__ float red[16];
    const int64_t c = threadIdx.x;
    const bool live = c * 8 < n;
    fused_u32x4_t v = {0u, 0u, 0u, 0u}, g = {0u, 0u, 0u, 0u};
    if (live) {
        v = *reinterpret_cast<const fused_u32x4_t*>(x + (int64_t)blockIdx.x * n + c * 8);
        g = *reinterpret_cast<const fused_u32x4_t*>(gamma + c * 8);
    }
    float f[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) { f[2 * i] = bf16lo(v[i]); f[2 * i + 1] = bf16hi(v[i]); }
    float q = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) q += f[i] * f[i];
    const float inv_rms = 1.0f / sqrtf(block_sum(q, red) * inv_n + eps);
    if (live) {
        fused_u32x4_t o;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            o[i] = pack_bf16x2((f[2 * i] * inv_rms) * bf16lo(g[i]), (f[2 * i + 1] * inv_rms) * bf16hi(g[i]));
        *reinterpret_cast<fused_u32x4_t*>(y + (int64_t)blockIdx.x * n + c * 8) = o;
    }
}
static bool aligned16(const void* a, const void* b, const void* c) {
    return (((uintptr_t)a | (uintptr_t)b | (uintptr_t)c) & 15u) == 0;
}
template <typename T>
static void rms_norm_t(hipStream_t s, const T* x, const T* g, T* y, int64_t rows, int64_t n, float inv_n, float eps) {
    if (sizeof(T) == 2 && n % 8 == 0 && n <= 8192 && aligned16(x, g, y)) {
        const int threads = (int)(cdiv(n / 8, 64) * 64);
        rms_norm_vec_kernel<<<(unsigned)rows, threads, 0, s>>>((const bf16_t*)x, (const bf16_t*)g, (bf16_t*)y, n, inv_n, eps);
        return;
    }
    const int block = n <= 256 ? 64 : (n <= 1024 ? 256 : 1024);  // decode has ONE row: spread it over many lanes
    const int64_t per = cdiv(n, block);
    if (per <= 4) rms_norm_kernel<T, 4><<<(unsigned)rows, block, 0, s>>>(x, g, y, n, inv_n, eps);
    else if (per <= 16) rms_norm_kernel<T, 16><<<(unsigned)rows, block, 0, s>>>(x, g, y, n, inv_n, eps);
    else rms_norm_long_kernel<T><<<(unsigned)rows, 1024, 0, s>>>(x, g, y, n, inv_n, eps);
}
// f32 rows and gains, bf16 result: the f32 value of normalization.rs:183-217 rounded once (the pair
// Cast(bf16)(rms_norm(x)) of a bf16 model whose residual stream is f32).  Rows whose length is a multiple of 8: two
// 16-byte loads of x and of gamma and one 16-byte store per thread.
__global__ void rms_norm_f32_bf16_kernel(const float* __restrict__ x, const float* __restrict__ gamma, bf16_t* __restrict__ y,
                                         int64_t n, float inv_n, float eps) {
    __shared__ float red[16];
    const float* row = x + (int64_t)blockIdx.x * n;
    bf16_t* out = y + (int64_t)blockIdx.x * n;
    const bool vec = (n % 8) == 0 && ((((uintptr_t)x | (uintptr_t)gamma | (uintptr_t)y) & 15u) == 0);
    float q = 0.f;
    if (vec) {
        for (int64_t c = threadIdx.x; c * 8 < n; c += blockDim.x) {
            const float4 a = *reinterpret_cast<const float4*>(row + c * 8), b = *reinterpret_cast<const float4*>(row + c * 8 + 4);
            q += a.x * a.x; q += a.y * a.y; q += a.z * a.z; q += a.w * a.w;
            q += b.x * b.x; q += b.y * b.y; q += b.z * b.z; q += b.w * b.w;
        }
    } else {
        for (int64_t i = threadIdx.x; i < n; i += blockDim.x) { const float v = row[i]; q += v * v; }
    }
    const float inv_rms = 1.0f / sqrtf(block_sum(q, red) * inv_n + eps);
    if (vec) {
        for (int64_t c = threadIdx.x; c * 8 < n; c += blockDim.x) {
            const float4 a = *reinterpret_cast<const float4*>(row + c * 8), b = *reinterpret_cast<const float4*>(row + c * 8 + 4);
            const float4 ga = *reinterpret_cast<const float4*>(gamma + c * 8), gb = *reinterpret_cast<const float4*>(gamma + c * 8 + 4);
            fused_u32x4_t o;
            o[0] = pack_bf16x2((a.x * inv_rms) * ga.x, (a.y * inv_rms) * ga.y);
            o[1] = pack_bf16x2((a.z * inv_rms) * ga.z, (a.w * inv_rms) * ga.w);
            o[2] = pack_bf16x2((b.x * inv_rms) * gb.x, (b.y * inv_rms) * gb.y);
            o[3] = pack_bf16x2((b.z * inv_rms) * gb.z, (b.w * inv_rms) * gb.w);
            *reinterpret_cast<fused_u32x4_t*>(out + c * 8) = o;
        }
    } else {
        for (int64_t i = threadIdx.x; i < n; i += blockDim.x) out[i] = f32_to_bf16((row[i] * inv_rms) * gamma[i]);
    }
}
void rms_norm_f32_to_bf16(hipStream_t s, const void* x, const void* gamma, void* y, int64_t rows, int64_t n, float inv_n,
                          float eps) {
    if (rows <= 0 || n <= 0) return;
    const int64_t chunks = cdiv(n, 8);
    const int threads = chunks <= 64 ? 64 : (chunks <= 256 ? 256 : (chunks <= 512 ? 512 : 1024));
    rms_norm_f32_bf16_kernel<<<(unsigned)rows, threads, 0, s>>>((const float*)x, (const float*)gamma, (bf16_t*)y, n, inv_n, eps);
}
void rms_norm(hipStream_t s, int dtype, const void* x, const void* gamma, void* y, int64_t rows, int64_t n, float inv_n,
              float eps) {
    if (rows <= 0 || n <= 0) return;
    if (dtype == 0) rms_norm_t<float>(s, (const float*)x, (const float*)gamma, (float*)y, rows, n, inv_n, eps);
    else rms_norm_t<bf16_t>(s, (const bf16_t*)x, (const bf16_t*)gamma, (bf16_t*)y, rows, n, inv_n, eps);
}

// ------------------------------------------------------------------------------ softmax
// common.rs:22-31: e = exp(x - max); y = e / sum(e)   (true division)
template <typename T>
__global__ void softmax_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t n) {
    __shared__ float red[16];
    const T* row = x + (int64_t)blockIdx.x * n;
    T* out = y + (int64_t)blockIdx.x * n;
    float mx = -INFINITY;
    for (int64_t i = threadIdx.x; i < n; i += blockDim.x) mx = fmaxf(mx, ldf(row, i));
    mx = block_max(mx, red);
    float sum = 0.f;
    for (int64_t i = threadIdx.x; i < n; i += blockDim.x) sum += expf(ldf(row, i) - mx);
    sum = block_sum(sum, red);
    for (int64_t i = threadIdx.x; i < n; i += blockDim.x) stf(out, i, expf(ldf(row, i) - mx) / sum);
}
void softmax_rows(hipStream_t s, int dtype, const void* x, void* y, int64_t rows, int64_t n) {
    if (rows <= 0 || n <= 0) return;
    const int block = n <= 64 ? 64 : (n <= 2048 ? 256 : 1024);
    if (dtype == 0) softmax_kernel<float><<<(unsigned)rows, block, 0, s>>>((const float*)x, (float*)y, n);
    else softmax_kernel<bf16_t><<<(unsigned)rows, block, 0, s>>>((const bf16_t*)x, (bf16_t*)y, n);
}

// ------------------------------------------------------------------------------ activations
// activation.rs:96-113: (x*0.5) * (erf(x / sqrt2) + 1); the three literals come from the program
template <typename T>
__global__ void gelu_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t n, float half, float div, float one) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        const float v = ldf(x, i);
        stf(y, i, (v * half) * (erff(v / div) + one));
    }
}
void gelu(hipStream_t s, int dtype, const void* x, void* y, int64_t n, float half, float div, float one) {
    if (n <= 0) return;
    const unsigned g = (unsigned)(cdiv(n, 256) > 16384 ? 16384 : cdiv(n, 256));
    if (dtype == 0) gelu_kernel<float><<<g, 256, 0, s>>>((const float*)x, (float*)y, n, half, div, one);
    else gelu_kernel<bf16_t><<<g, 256, 0, s>>>((const bf16_t*)x, (bf16_t*)y, n, half, div, one);
}
// activation.rs:141-162: (g / (1 + exp(g * -1))) * u
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gate, const T* __restrict__ up, T* __restrict__ y, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        const float g = ldf(gate, i);
        float r = g / (1.0f + expf(g * -1.0f));
        if (up) r *= ldf(up, i);
        stf(y, i, r);
    }
}
void swiglu(hipStream_t s, int dtype, const void* gate, const void* up, void* y, int64_t n) {
    if (n <= 0) return;
    const unsigned g = (unsigned)(cdiv(n, 256) > 16384 ? 16384 : cdiv(n, 256));
    if (dtype == 0) swiglu_kernel<float><<<g, 256, 0, s>>>((const float*)gate, (const float*)up, (float*)y, n);
    else swiglu_kernel<bf16_t><<<g, 256, 0, s>>>((const bf16_t*)gate, (const bf16_t*)up, (bf16_t*)y, n);
}

// ------------------------------------------------------------------------------ RoPE
// rotary.rs:430-536 on packed rows [T, Q|K|V]: for each Q/K head and j < half:
//   out[j]      = a*cos[t,j] - b*sin[t,j]      (a = x[j], b = x[j+half])
//   out[j+half] = b*cos[t,j] + a*sin[t,j]
// columns >= 2*half of a head and all of V pass through.
template <typename T>
__global__ void rope_kernel(const T* __restrict__ qkv, const T* __restrict__ cs, const T* __restrict__ sn,
                            T* __restrict__ out, int64_t t, int64_t qk_cols, int64_t total_cols, int64_t head_dim,
                            int64_t half) {
    const int64_t total = t * total_cols;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t row = idx / total_cols, col = idx % total_cols;
        float r;
        if (col < qk_cols) {
            const int64_t d = col % head_dim;
            if (d < half) {
                const float a = ldf(qkv, idx), b = ldf(qkv, idx + half);
                r = a * ldf(cs, row * half + d) - b * ldf(sn, row * half + d);
            } else if (d < 2 * half) {
                const int64_t j = d - half;
                const float b = ldf(qkv, idx), a = ldf(qkv, idx - half);
                r = b * ldf(cs, row * half + j) + a * ldf(sn, row * half + j);
            } else {
                r = ldf(qkv, idx);
            }
        } else {
            r = ldf(qkv, idx);
        }
        stf(out, idx, r);
    }
}
// bf16 with head_dim = 2 half and half a multiple of 8: a thread produces 8 consecutive outputs (16 bytes) from 16-byte
// loads of the two halves of the head and of the tables; V chunks pass through.
__global__ __launch_bounds__(256) void rope_vec_kernel(const bf16_t* __restrict__ qkv, const bf16_t* __restrict__ cs,
                                                       const bf16_t* __restrict__ sn, bf16_t* __restrict__ out, int64_t chunks,
                                                       int row_chunks, int qk_chunks, int head_chunks) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= chunks) return;
    const int64_t row = idx / row_chunks;
    const int c = (int)(idx % row_chunks);
    const fused_u32x4_t own = *reinterpret_cast<const fused_u32x4_t*>(qkv + idx * 8);
    fused_u32x4_t o = own;
    if (c < qk_chunks) {
        const int half_chunks = head_chunks / 2;
        const int d = c % head_chunks;
        const bool second = d >= half_chunks;
        const int j = second ? d - half_chunks : d;
        const fused_u32x4_t other = *reinterpret_cast<const fused_u32x4_t*>(qkv + (idx + (second ? -half_chunks : half_chunks)) * 8);
        const fused_u32x4_t cv = *reinterpret_cast<const fused_u32x4_t*>(cs + (row * half_chunks + j) * 8);
        const fused_u32x4_t sv = *reinterpret_cast<const fused_u32x4_t*>(sn + (row * half_chunks + j) * 8);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float r[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const float mine = h ? bf16hi(own[i]) : bf16lo(own[i]);
                const float oth = h ? bf16hi(other[i]) : bf16lo(other[i]);
                const float cc = h ? bf16hi(cv[i]) : bf16lo(cv[i]);
                const float ss = h ? bf16hi(sv[i]) : bf16lo(sv[i]);
                // first half: a cos - b sin with a = mine, b = oth; second half: b cos + a sin with b = mine, a = oth
                r[h] = second ? mine * cc + oth * ss : mine * cc - oth * ss;
            }
            o[i] = pack_bf16x2(r[0], r[1]);
        }
    }
    *reinterpret_cast<fused_u32x4_t*>(out + idx * 8) = o;
}
void rope_packed(hipStream_t s, int dtype, const void* qkv, const void* cos, const void* sin, void* out, int64_t t,
                 int64_t n_q, int64_t n_kv, int64_t head_dim, int64_t half) {
    const int64_t qk_cols = (n_q + n_kv) * head_dim, total_cols = (n_q + 2 * n_kv) * head_dim;
    const int64_t total = t * total_cols;
    if (total <= 0) return;
    const unsigned g = (unsigned)(cdiv(total, 256) > 16384 ? 16384 : cdiv(total, 256));
    if (dtype != 0 && head_dim == 2 * half && half % 8 == 0 && aligned16(qkv, out, cos) && aligned16(sin, sin, sin) &&
        cdiv(total / 8, 256) < (1ll << 31)) {
        const int64_t chunks = total / 8;
        rope_vec_kernel<<<(unsigned)cdiv(chunks, 256), 256, 0, s>>>((const bf16_t*)qkv, (const bf16_t*)cos, (const bf16_t*)sin, (bf16_t*)out,
                                                                     chunks, (int)(total_cols / 8), (int)(qk_cols / 8), (int)(head_dim / 8));
        return;
    }
    if (dtype == 0)
        rope_kernel<float><<<g, 256, 0, s>>>((const float*)qkv, (const float*)cos, (const float*)sin, (float*)out, t, qk_cols, total_cols, head_dim, half);
    else
        rope_kernel<bf16_t><<<g, 256, 0, s>>>((const bf16_t*)qkv, (const bf16_t*)cos, (const bf16_t*)sin, (bf16_t*)out, t, qk_cols, total_cols, head_dim, half);
}

}  // namespace k
}  // namespace gptrs
