// Weight-only quantisation: int8 per output channel and int4 in groups of 128 along K, both symmetric.
// Build-defined extension ops (the reference leaves Quantize/Dequantize "backend-defined",
// docs/backend.md:620-632, and its CPU backend answers Unimplemented, cpu.rs:326-331).  Quantisers are
// written so that every f32 operation (max, IEEE division, round-half-even, clamp) is the one numpy
// performs in the closed form the tests hold, hence bit-identical packs.
#include "kernels.hpp"
#include "device_utils.hpp"

namespace gptrs {
namespace k {

namespace {

template <typename T> __device__ __forceinline__ float ldw(const T* p, int64_t i);
template <> __device__ __forceinline__ float ldw<float>(const float* p, int64_t i) { return p[i]; }
template <> __device__ __forceinline__ float ldw<bf16_t>(const bf16_t* p, int64_t i) { return bf16_to_f32(p[i]); }
template <typename T> __device__ __forceinline__ void stw(T* p, int64_t i, float v);
template <> __device__ __forceinline__ void stw<float>(float* p, int64_t i, float v) { p[i] = v; }
template <> __device__ __forceinline__ void stw<bf16_t>(bf16_t* p, int64_t i, float v) { p[i] = f32_to_bf16(v); }
__device__ __forceinline__ float rbf16(float v) { return bf16_to_f32(f32_to_bf16(v)); }

// scales[g][n] = bf16(max_{k in group g} |w[k][n]| / qmax), 1 where that is 0; one thread per (g, n)
template <typename T>
__global__ void scales_kernel(const T* __restrict__ w, T* __restrict__ scales, int64_t K, int64_t N, int64_t group, float qmax) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t ngroups = K / group;
    if (idx >= ngroups * N) return;
    const int64_t g = idx / N, n = idx % N;
    float amax = 0.f;
    for (int64_t kk = g * group; kk < (g + 1) * group; ++kk) amax = fmaxf(amax, fabsf(ldw(w, kk * N + n)));
    float s = rbf16(amax / qmax);
    if (s == 0.f) s = 1.0f;
    stw(scales, idx, s);
}
// The same for ONE group (the whole column, int8): a thread per column is a few dozen waves walking K one row at a time, so
// a workgroup of 16 waves takes 64 columns, wave y the rows y, y + 16, ..., and the 16 maxima of a column meet in LDS
// (a maximum does not depend on the order it is taken in).
template <typename T>
__global__ __launch_bounds__(1024) void column_scales_kernel(const T* __restrict__ w, T* __restrict__ scales, int64_t K, int64_t N, float qmax) {
    __shared__ float part[16][64];
    const int c = threadIdx.x & 63, y = threadIdx.x >> 6;
    const int64_t n = (int64_t)blockIdx.x * 64 + c;
    float amax = 0.f;
    if (n < N) {
        int64_t kk = y;
        for (; kk + 48 < K; kk += 64) {   // four rows in flight
            const float a = fabsf(ldw(w, kk * N + n)), b = fabsf(ldw(w, (kk + 16) * N + n));
            const float d = fabsf(ldw(w, (kk + 32) * N + n)), e = fabsf(ldw(w, (kk + 48) * N + n));
            amax = fmaxf(fmaxf(amax, fmaxf(a, b)), fmaxf(d, e));
        }
        for (; kk < K; kk += 16) amax = fmaxf(amax, fabsf(ldw(w, kk * N + n)));
    }
    part[y][c] = amax;
    __syncthreads();
    if (y == 0 && n < N) {
#pragma unroll
        for (int i = 1; i < 16; ++i) amax = fmaxf(amax, part[i][c]);
        float s = rbf16(amax / qmax);
        if (s == 0.f) s = 1.0f;
        stw(scales, n, s);
    }
}
template <typename T>
__global__ void quant_w8_kernel(const T* __restrict__ w, const T* __restrict__ scales, int8_t* __restrict__ q, int64_t K, int64_t N) {
    const int64_t total = K * N;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        const float v = rintf(ldw(w, i) / ldw(scales, i % N));
        q[i] = (int8_t)fminf(fmaxf(v, -127.f), 127.f);
    }
}
template <typename T>
__global__ void quant_w4_kernel(const T* __restrict__ w, const T* __restrict__ scales, uint8_t* __restrict__ packed, int64_t K, int64_t N) {
    const int64_t total = (K / 2) * N;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t k2 = i / N, n = i % N;
        const float s = ldw(scales, ((2 * k2) / 128) * N + n);
        const float a = fminf(fmaxf(rintf(ldw(w, (2 * k2) * N + n) / s), -7.f), 7.f);
        const float b = fminf(fmaxf(rintf(ldw(w, (2 * k2 + 1) * N + n) / s), -7.f), 7.f);
        packed[i] = (uint8_t)(((int)a & 0xF) | (((int)b & 0xF) << 4));
    }
}
template <typename T>
__global__ void dequant_w8_kernel(const int8_t* __restrict__ q, const T* __restrict__ scales, T* __restrict__ out, int64_t K, int64_t N) {
    const int64_t total = K * N;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x)
        stw(out, i, (float)q[i] * ldw(scales, i % N));
}
template <typename T>
__global__ void dequant_w4_kernel(const uint8_t* __restrict__ packed, const T* __restrict__ scales, T* __restrict__ out, int64_t K, int64_t N) {
    const int64_t total = (K / 2) * N;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t k2 = i / N, n = i % N;
        const float s = ldw(scales, ((2 * k2) / 128) * N + n);
        const int b = packed[i];
        int lo = b & 0xF, hi = b >> 4;
        if (lo > 7) lo -= 16;
        if (hi > 7) hi -= 16;
        stw(out, (2 * k2) * N + n, (float)lo * s);
        stw(out, (2 * k2 + 1) * N + n, (float)hi * s);
    }
}

inline unsigned grid_for(int64_t total) {
    const int64_t g = (total + 255) / 256;
    return (unsigned)(g < 1 ? 1 : (g > 65536 ? 65536 : g));
}

}  // namespace

#define GPTRS_BY_DTYPE(CALL_F32, CALL_BF16) do { if (dtype == 0) { CALL_F32; } else { CALL_BF16; } } while (0)

void quant_w8_scales(hipStream_t s, int dtype, const void* w, void* scales, int64_t k, int64_t n) {
    if (k <= 0 || n <= 0) return;
    const unsigned blocks = (unsigned)((n + 63) / 64);
    GPTRS_BY_DTYPE((column_scales_kernel<float><<<blocks, 1024, 0, s>>>((const float*)w, (float*)scales, k, n, 127.0f)),
                   (column_scales_kernel<bf16_t><<<blocks, 1024, 0, s>>>((const bf16_t*)w, (bf16_t*)scales, k, n, 127.0f)));
}
void quant_w8(hipStream_t s, int dtype, const void* w, const void* scales, int8_t* q, int64_t k, int64_t n) {
    if (k <= 0 || n <= 0) return;
    GPTRS_BY_DTYPE((quant_w8_kernel<float><<<grid_for(k * n), 256, 0, s>>>((const float*)w, (const float*)scales, q, k, n)),
                   (quant_w8_kernel<bf16_t><<<grid_for(k * n), 256, 0, s>>>((const bf16_t*)w, (const bf16_t*)scales, q, k, n)));
}
void quant_w4g128_scales(hipStream_t s, int dtype, const void* w, void* scales, int64_t k, int64_t n) {
    if (k <= 0 || n <= 0) return;
    GPTRS_BY_DTYPE((scales_kernel<float><<<grid_for(k / 128 * n), 256, 0, s>>>((const float*)w, (float*)scales, k, n, 128, 7.0f)),
                   (scales_kernel<bf16_t><<<grid_for(k / 128 * n), 256, 0, s>>>((const bf16_t*)w, (bf16_t*)scales, k, n, 128, 7.0f)));
}
void quant_w4g128(hipStream_t s, int dtype, const void* w, const void* scales, uint8_t* packed, int64_t k, int64_t n) {
    if (k <= 0 || n <= 0) return;
    GPTRS_BY_DTYPE((quant_w4_kernel<float><<<grid_for(k / 2 * n), 256, 0, s>>>((const float*)w, (const float*)scales, packed, k, n)),
                   (quant_w4_kernel<bf16_t><<<grid_for(k / 2 * n), 256, 0, s>>>((const bf16_t*)w, (const bf16_t*)scales, packed, k, n)));
}
void dequant_w8(hipStream_t s, int dtype, const int8_t* q, const void* scales, void* out, int64_t k, int64_t n) {
    if (k <= 0 || n <= 0) return;
    GPTRS_BY_DTYPE((dequant_w8_kernel<float><<<grid_for(k * n), 256, 0, s>>>(q, (const float*)scales, (float*)out, k, n)),
                   (dequant_w8_kernel<bf16_t><<<grid_for(k * n), 256, 0, s>>>(q, (const bf16_t*)scales, (bf16_t*)out, k, n)));
}
void dequant_w4g128(hipStream_t s, int dtype, const uint8_t* packed, const void* scales, void* out, int64_t k, int64_t n) {
    if (k <= 0 || n <= 0) return;
    GPTRS_BY_DTYPE((dequant_w4_kernel<float><<<grid_for(k / 2 * n), 256, 0, s>>>(packed, (const float*)scales, (float*)out, k, n)),
                   (dequant_w4_kernel<bf16_t><<<grid_for(k / 2 * n), 256, 0, s>>>(packed, (const bf16_t*)scales, (bf16_t*)out, k, n)));
}
#undef GPTRS_BY_DTYPE

}  // namespace k
}  // namespace gptrs
