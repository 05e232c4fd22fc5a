// One generic kernel per PTIR op family: the executor's "fusion off" path and the fallback for
// every instruction no fused kernel claims.  Semantics follow the reference interpreter
// (crates/gpt-rs-backend-ref-cpu/src/cpu.rs) and docs/backend.md; integer / index ops are
// bit-exact, float ops compute in f32 and round once to the output dtype.
#include <cstring>

#include <mutex>

#include "kernels.hpp"
#include "device_utils.hpp"

namespace gptrs {
namespace k {

static inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }
static inline unsigned grid_for(int64_t n, int block, int64_t cap = 1 << 20) {
    int64_t g = cdiv(n, block);
    if (g < 1) g = 1;
    if (g > cap) g = cap;
    return (unsigned)g;
}

// ------------------------------------------------------------------------------ strided copy
template <typename T>
__global__ void copy_strided_kernel(T* __restrict__ dst, const T* __restrict__ src, CopyDesc d,
                                    const int32_t* __restrict__ starts) {
    int64_t dyn_off = 0;
    if (d.dyn) {
        for (int i = 0; i < d.dyn_rank; ++i) {
            int64_t s = starts[i];
            s = s < 0 ? 0 : s;
            s = s > d.dyn_max[i] ? d.dyn_max[i] : s;
            dyn_off += s * d.dyn_stride[i];
        }
    }
    const int64_t src_base = d.src_off + (d.dyn == 1 ? dyn_off : 0);
    const int64_t dst_base = d.dst_off + (d.dyn == 2 ? dyn_off : 0);
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < d.total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        int64_t rem = idx, so = src_base, dof = dst_base;
#pragma unroll
        for (int i = kMaxRank - 1; i >= 0; --i) {
            if (i < d.rank) {
                const int64_t c = rem % d.dims[i];
                rem /= d.dims[i];
                so += c * d.src_stride[i];
                dof += c * d.dst_stride[i];
            }
        }
        dst[dof] = src[so];
    }
}

void copy_strided(hipStream_t s, void* dst, const void* src, int elem_size, const CopyDesc& d, const int32_t* starts) {
    if (d.total <= 0) return;
    const int block = 256;
    const unsigned grid = grid_for(d.total, block, 65536);
    switch (elem_size) {
        case 1: copy_strided_kernel<uint8_t><<<grid, block, 0, s>>>((uint8_t*)dst, (const uint8_t*)src, d, starts); break;
        case 2: copy_strided_kernel<uint16_t><<<grid, block, 0, s>>>((uint16_t*)dst, (const uint16_t*)src, d, starts); break;
        case 4: copy_strided_kernel<uint32_t><<<grid, block, 0, s>>>((uint32_t*)dst, (const uint32_t*)src, d, starts); break;
        case 8: copy_strided_kernel<uint64_t><<<grid, block, 0, s>>>((uint64_t*)dst, (const uint64_t*)src, d, starts); break;
        case 16: copy_strided_kernel<uint4><<<grid, block, 0, s>>>((uint4*)dst, (const uint4*)src, d, starts); break;
        default: break;
    }
}

__global__ void store_small_kernel(uint8_t* dst, SmallPayload p, int nbytes) {
    const int i = threadIdx.x;
    if (i < nbytes) dst[i] = ((const uint8_t*)p.w)[i];
}
void store_small(hipStream_t s, void* dst, const SmallPayload& p, int nbytes) {
    if (nbytes <= 0) return;
    store_small_kernel<<<1, 256, 0, s>>>((uint8_t*)dst, p, nbytes);
}

__global__ void fill_zero_kernel(uint4* dst, int64_t n16, uint8_t* tail, int ntail) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (int64_t)gridDim.x * blockDim.x)
        dst[i] = make_uint4(0, 0, 0, 0);
    if (blockIdx.x == 0 && (int)threadIdx.x < ntail) tail[threadIdx.x] = 0;
}
void fill_zero(hipStream_t s, void* dst, size_t nbytes) {
    if (!nbytes) return;
    const int64_t n16 = (int64_t)(nbytes / 16);
    fill_zero_kernel<<<grid_for(n16 ? n16 : 1, 256, 8192), 256, 0, s>>>((uint4*)dst, n16, (uint8_t*)dst + n16 * 16,
                                                                          (int)(nbytes % 16));
}

// ------------------------------------------------------------------------------ elementwise
template <typename T> __device__ __forceinline__ float ldf(const T* p, int64_t i);
template <> __device__ __forceinline__ float ldf<float>(const float* p, int64_t i) { return p[i]; }
template <> __device__ __forceinline__ float ldf<bf16_t>(const bf16_t* p, int64_t i) { return bf16_to_f32(p[i]); }
template <typename T> __device__ __forceinline__ void stf(T* p, int64_t i, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, int64_t i, float v) { p[i] = v; }
template <> __device__ __forceinline__ void stf<bf16_t>(bf16_t* p, int64_t i, float v) { p[i] = f32_to_bf16(v); }

__device__ __forceinline__ float apply_unary(int op, float v) {
    switch (op) {  // cpu.rs:1704-1714
        case 0: return -v;
        case 1: return fabsf(v);
        case 2: return expf(v);
        case 3: return logf(v);
        case 4: return tanhf(v);
        case 5: return erff(v);
        case 6: return 1.0f / sqrtf(v);
        default: return 1.0f / v;
    }
}
__device__ __forceinline__ float apply_binary(int op, float a, float b) {
    switch (op) {  // cpu.rs:1669-1677; Rust max/min return the non-NaN operand == fmaxf/fminf
        case 0: return a + b;
        case 1: return a - b;
        case 2: return a * b;
        case 3: return a / b;
        case 4: return fmaxf(a, b);
        default: return fminf(a, b);
    }
}

template <typename T>
__global__ void unary_kernel(int op, const T* __restrict__ x, T* __restrict__ y, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        stf(y, i, apply_unary(op, ldf(x, i)));
}
template <typename T>
__global__ void binary_kernel(int op, const T* __restrict__ a, const T* __restrict__ b, T* __restrict__ y, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        stf(y, i, apply_binary(op, ldf(a, i), ldf(b, i)));
}
template <typename T>
__global__ void binary_scalar_kernel(int op, const T* __restrict__ a, float b, T* __restrict__ y, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        stf(y, i, apply_binary(op, ldf(a, i), b));
}

void unary(hipStream_t s, int dtype, int op, const void* x, void* y, int64_t n) {
    if (n <= 0) return;
    if (dtype == 0) unary_kernel<float><<<grid_for(n, 256, 16384), 256, 0, s>>>(op, (const float*)x, (float*)y, n);
    else unary_kernel<bf16_t><<<grid_for(n, 256, 16384), 256, 0, s>>>(op, (const bf16_t*)x, (bf16_t*)y, n);
}
void binary(hipStream_t s, int dtype, int op, const void* a, const void* b, void* y, int64_t n) {
    if (n <= 0) return;
    if (dtype == 0) binary_kernel<float><<<grid_for(n, 256, 16384), 256, 0, s>>>(op, (const float*)a, (const float*)b, (float*)y, n);
    else binary_kernel<bf16_t><<<grid_for(n, 256, 16384), 256, 0, s>>>(op, (const bf16_t*)a, (const bf16_t*)b, (bf16_t*)y, n);
}
void binary_scalar(hipStream_t s, int dtype, int op, const void* a, float b, void* y, int64_t n) {
    if (n <= 0) return;
    if (dtype == 0) binary_scalar_kernel<float><<<grid_for(n, 256, 16384), 256, 0, s>>>(op, (const float*)a, b, (float*)y, n);
    else binary_scalar_kernel<bf16_t><<<grid_for(n, 256, 16384), 256, 0, s>>>(op, (const bf16_t*)a, b, (bf16_t*)y, n);
}

template <typename T>
__device__ __forceinline__ bool cmp_apply(int op, T x, T y) {
    switch (op) {  // cpu.rs:2254-2261; float NaN rules are IEEE (docs/backend.md:199-202)
        case 0: return x < y;
        case 1: return x <= y;
        case 2: return x == y;
        case 3: return x >= y;
        case 4: return x > y;
        default: return x != y;
    }
}
__global__ void compare_i32_kernel(int op, const int32_t* a, const int32_t* b, uint8_t* y, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        y[i] = cmp_apply<int32_t>(op, a[i], b[i]) ? 1 : 0;
}
template <typename T>
__global__ void compare_f_kernel(int op, const T* a, const T* b, uint8_t* y, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        y[i] = cmp_apply<float>(op, ldf(a, i), ldf(b, i)) ? 1 : 0;
}
void compare(hipStream_t s, int dtype, int op, const void* a, const void* b, uint8_t* y, int64_t n) {
    if (n <= 0) return;
    const unsigned g = grid_for(n, 256, 16384);
    if (dtype == 3) compare_i32_kernel<<<g, 256, 0, s>>>(op, (const int32_t*)a, (const int32_t*)b, y, n);
    else if (dtype == 0) compare_f_kernel<float><<<g, 256, 0, s>>>(op, (const float*)a, (const float*)b, y, n);
    else compare_f_kernel<bf16_t><<<g, 256, 0, s>>>(op, (const bf16_t*)a, (const bf16_t*)b, y, n);
}

template <typename T>
__global__ void select_kernel(const uint8_t* p, const T* t, const T* f, T* y, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        y[i] = p[i] != 0 ? t[i] : f[i];
}
void select(hipStream_t s, int elem_size, const uint8_t* p, const void* t, const void* f, void* y, int64_t n) {
    if (n <= 0) return;
    const unsigned g = grid_for(n, 256, 16384);
    if (elem_size == 4) select_kernel<uint32_t><<<g, 256, 0, s>>>(p, (const uint32_t*)t, (const uint32_t*)f, (uint32_t*)y, n);
    else if (elem_size == 2) select_kernel<uint16_t><<<g, 256, 0, s>>>(p, (const uint16_t*)t, (const uint16_t*)f, (uint16_t*)y, n);
    else select_kernel<uint8_t><<<g, 256, 0, s>>>(p, (const uint8_t*)t, (const uint8_t*)f, (uint8_t*)y, n);
}

// cast (docs/backend.md:96-102; cpu.rs:1472-1583).  Source value is first widened to
// (is_int ? int32 : float); destination rules: float->int trunc + saturate, NaN -> 0;
// ->i1 is (x != 0); int->float nearest; float->float RNE.
__device__ __forceinline__ int32_t f32_to_i32_sat(float v) {
    if (v != v) return 0;
    const float t = truncf(v);
    if (t >= 2147483648.0f) return 2147483647;
    if (t <= -2147483648.0f) return (int32_t)0x80000000;
    return (int32_t)t;
}
__global__ void cast_kernel(int sd, int dd, const void* x, void* y, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        float fv = 0.f;
        int32_t iv = 0;
        bool is_int = false;
        switch (sd) {
            case 0: fv = ((const float*)x)[i]; break;
            case 2: fv = bf16_to_f32(((const bf16_t*)x)[i]); break;
            case 3: iv = ((const int32_t*)x)[i]; is_int = true; break;
            case 4: iv = ((const uint8_t*)x)[i] != 0 ? 1 : 0; is_int = true; break;
            case 5: iv = ((const int8_t*)x)[i]; is_int = true; break;
            default: iv = ((const uint8_t*)x)[i]; is_int = true; break;
        }
        switch (dd) {
            case 0: ((float*)y)[i] = is_int ? (float)iv : fv; break;
            case 2: ((bf16_t*)y)[i] = f32_to_bf16(is_int ? (float)iv : fv); break;
            case 3: ((int32_t*)y)[i] = is_int ? iv : f32_to_i32_sat(fv); break;
            case 4: ((uint8_t*)y)[i] = is_int ? (iv != 0) : (fv != 0.0f); break;
            case 5: {
                int32_t v = is_int ? iv : f32_to_i32_sat(fv);
                ((int8_t*)y)[i] = (int8_t)(v < -128 ? -128 : (v > 127 ? 127 : v));
                break;
            }
            default: {
                int32_t v = is_int ? iv : f32_to_i32_sat(fv);
                ((uint8_t*)y)[i] = (uint8_t)(v < 0 ? 0 : (v > 255 ? 255 : v));
                break;
            }
        }
    }
}
void cast(hipStream_t s, int sd, int dd, const void* x, void* y, int64_t n) {
    if (n <= 0) return;
    cast_kernel<<<grid_for(n, 256, 16384), 256, 0, s>>>(sd, dd, x, y, n);
}

__global__ void iota_kernel(int32_t* y, int64_t total, int64_t axis_len, int64_t inner) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x)
        y[i] = (int32_t)((i / inner) % axis_len);
}
void iota(hipStream_t s, int32_t* y, int64_t outer, int64_t axis_len, int64_t inner) {
    const int64_t total = outer * axis_len * inner;
    if (total <= 0) return;
    iota_kernel<<<grid_for(total, 256, 16384), 256, 0, s>>>(y, total, axis_len, inner);
}

// ------------------------------------------------------------------------------ reduce
__device__ __forceinline__ float red_id(int kind) { return kind == 0 ? 0.f : (kind == 1 ? -INFINITY : INFINITY); }
__device__ __forceinline__ float red_op(int kind, float a, float b) {
    return kind == 0 ? a + b : (kind == 1 ? fmaxf(a, b) : fminf(a, b));
}

// inner == 1: one 256-thread block per row, wave64 shuffle tree then LDS across waves.
template <typename T>
__global__ void reduce_rows_kernel(int kind, const T* __restrict__ x, T* __restrict__ y, int64_t n) {
    __shared__ float part[4];
    const T* row = x + (int64_t)blockIdx.x * n;
    float acc = red_id(kind);
    for (int64_t i = threadIdx.x; i < n; i += blockDim.x) acc = red_op(kind, acc, ldf(row, i));
    for (int off = 32; off > 0; off >>= 1) acc = red_op(kind, acc, __shfl_down(acc, off, 64));
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        float r = part[0];
        for (int w = 1; w < (int)(blockDim.x >> 6); ++w) r = red_op(kind, r, part[w]);
        stf(y, (int64_t)blockIdx.x, r);
    }
}
// inner > 1: one thread per (outer, inner) column, sequential over the axis (coalesced across inner).
template <typename T>
__global__ void reduce_cols_kernel(int kind, const T* __restrict__ x, T* __restrict__ y, int64_t outer,
                                   int64_t axis_len, int64_t inner) {
    const int64_t total = outer * inner;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t o = idx / inner, i = idx % inner;
        const T* base = x + o * axis_len * inner + i;
        float acc = red_id(kind);
        for (int64_t a = 0; a < axis_len; ++a) acc = red_op(kind, acc, ldf(base, a * inner));
        stf(y, idx, acc);
    }
}
void reduce(hipStream_t s, int dtype, int kind, const void* x, void* y, int64_t outer, int64_t axis_len, int64_t inner) {
    if (outer * inner <= 0) return;
    if (inner == 1) {
        if (dtype == 0) reduce_rows_kernel<float><<<(unsigned)outer, 256, 0, s>>>(kind, (const float*)x, (float*)y, axis_len);
        else reduce_rows_kernel<bf16_t><<<(unsigned)outer, 256, 0, s>>>(kind, (const bf16_t*)x, (bf16_t*)y, axis_len);
    } else {
        const unsigned g = grid_for(outer * inner, 256, 16384);
        if (dtype == 0) reduce_cols_kernel<float><<<g, 256, 0, s>>>(kind, (const float*)x, (float*)y, outer, axis_len, inner);
        else reduce_cols_kernel<bf16_t><<<g, 256, 0, s>>>(kind, (const bf16_t*)x, (bf16_t*)y, outer, axis_len, inner);
    }
}

// ------------------------------------------------------------------------------ take
template <typename T>
__global__ void take_kernel(const T* __restrict__ table, const int32_t* __restrict__ idx, T* __restrict__ y,
                            int64_t vocab, int64_t inner, int* err_flag) {
    const int64_t r = blockIdx.x;
    const int32_t id = idx[r];
    const bool ok = id >= 0 && (int64_t)id < vocab;
    if (!ok && threadIdx.x == 0) atomicExch(err_flag, 1);
    const T* src = table + (int64_t)(ok ? id : 0) * inner;
    T* dst = y + r * inner;
    for (int64_t i = threadIdx.x; i < inner; i += blockDim.x) dst[i] = ok ? src[i] : T{};
}
void take(hipStream_t s, int elem_size, const void* table, const int32_t* idx, void* y, int64_t n_idx, int64_t vocab,
          int64_t inner, int* err_flag) {
    if (n_idx <= 0 || inner <= 0) return;
    // widen to 16/8/4-byte words when the row allows it
    const size_t row_bytes = (size_t)inner * elem_size;
    const bool a16 = row_bytes % 16 == 0 && ((uintptr_t)table % 16 == 0) && ((uintptr_t)y % 16 == 0);
    if (a16) {
        take_kernel<uint4><<<(unsigned)n_idx, 256, 0, s>>>((const uint4*)table, idx, (uint4*)y, vocab, (int64_t)(row_bytes / 16), err_flag);
    } else if (elem_size == 4) {
        take_kernel<uint32_t><<<(unsigned)n_idx, 256, 0, s>>>((const uint32_t*)table, idx, (uint32_t*)y, vocab, inner, err_flag);
    } else if (elem_size == 2) {
        take_kernel<uint16_t><<<(unsigned)n_idx, 256, 0, s>>>((const uint16_t*)table, idx, (uint16_t*)y, vocab, inner, err_flag);
    } else {
        take_kernel<uint8_t><<<(unsigned)n_idx, 256, 0, s>>>((const uint8_t*)table, idx, (uint8_t*)y, vocab, inner, err_flag);
    }
}

// ------------------------------------------------------------------------------ generic dot
// 32x32 output tile per 256-thread block, K stepped by 32 through LDS; arbitrary operand strides.
// Correctness path for dots no tuned kernel claims (attention score / PV contractions in prefill,
// odd shapes).  Accumulates in f32 in k order within a tile.
template <typename T, typename TO>
__global__ void dot_generic_kernel(const T* __restrict__ a, const T* __restrict__ b, TO* __restrict__ c, DotDesc d) {
    __shared__ float As[32][33];
    __shared__ float Bs[32][33];
    const int64_t bi = blockIdx.z;
    const int64_t m0 = (int64_t)blockIdx.y * 32, n0 = (int64_t)blockIdx.x * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // ty in 0..7
    const T* ab = a + bi * d.a_sb;
    const T* bb = b + bi * d.b_sb;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int64_t k0 = 0; k0 < d.k; k0 += 32) {
        for (int r = ty; r < 32; r += 8) {
            const int64_t m = m0 + r, kk = k0 + tx;
            As[r][tx] = (m < d.m && kk < d.k) ? ldf(ab, m * d.a_sm + kk * d.a_sk) : 0.f;
            const int64_t kr = k0 + r, n = n0 + tx;
            Bs[r][tx] = (kr < d.k && n < d.n) ? ldf(bb, kr * d.b_sk + n * d.b_sn) : 0.f;
        }
        __syncthreads();
#pragma unroll 8
        for (int kk = 0; kk < 32; ++kk) {
            const float bv = Bs[kk][tx];
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[j] += As[ty + 8 * j][kk] * bv;
        }
        __syncthreads();
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int64_t m = m0 + ty + 8 * j, n = n0 + tx;
        if (m < d.m && n < d.n) stf(c, bi * d.c_sb + m * d.c_sm + n, acc[j]);
    }
}
void dot_generic(hipStream_t s, int dtype, const void* a, const void* b, void* c, const DotDesc& d, bool out_f32) {
    if (d.batch * d.m * d.n <= 0) return;
    dim3 grid((unsigned)cdiv(d.n, 32), (unsigned)cdiv(d.m, 32), (unsigned)d.batch);
    if (dtype == 0) dot_generic_kernel<float, float><<<grid, 256, 0, s>>>((const float*)a, (const float*)b, (float*)c, d);
    else if (out_f32) dot_generic_kernel<bf16_t, float><<<grid, 256, 0, s>>>((const bf16_t*)a, (const bf16_t*)b, (float*)c, d);
    else dot_generic_kernel<bf16_t, bf16_t><<<grid, 256, 0, s>>>((const bf16_t*)a, (const bf16_t*)b, (bf16_t*)c, d);
}

// ------------------------------------------------------------------------------ sampling
// argmax of the last row: stage 1 = per-block (value, smallest index) partials, stage 2 = one
// block combines.  Ties -> smallest index (docs/backend.md:270).
template <typename T>
__global__ void argmax_stage1(const T* __restrict__ row, int64_t n, float* pv, int32_t* pi) {
    __shared__ float sv[4];
    __shared__ int32_t si[4];
    float best = -INFINITY;
    int32_t bidx = 0x7fffffff;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        const float v = ldf(row, i);
        if (v > best || (v == best && (int32_t)i < bidx)) { best = v; bidx = (int32_t)i; }
    }
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_down(best, off, 64);
        const int32_t oi = __shfl_down(bidx, off, 64);
        if (ov > best || (ov == best && oi < bidx)) { best = ov; bidx = oi; }
    }
    if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = best; si[threadIdx.x >> 6] = bidx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; ++w)
            if (sv[w] > best || (sv[w] == best && si[w] < bidx)) { best = sv[w]; bidx = si[w]; }
        pv[blockIdx.x] = best;
        pi[blockIdx.x] = bidx;
    }
}
__global__ void argmax_stage2(const float* pv, const int32_t* pi, int nparts, int64_t* out) {
    float best = -INFINITY;
    int32_t bidx = 0x7fffffff;
    for (int i = threadIdx.x; i < nparts; i += 64) {
        const float v = pv[i];
        const int32_t id = pi[i];
        if (v > best || (v == best && id < bidx)) { best = v; bidx = id; }
    }
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_down(best, off, 64);
        const int32_t oi = __shfl_down(bidx, off, 64);
        if (ov > best || (ov == best && oi < bidx)) { best = ov; bidx = oi; }
    }
    if (threadIdx.x == 0) *out = bidx == 0x7fffffff ? 0 : (int64_t)bidx;
}
void argmax_last_row(hipStream_t s, int dtype, const void* logits, int64_t rows, int64_t vocab, int64_t* out,
                     float* scratch_val, int32_t* scratch_idx, int scratch_cap) {
    int nb = (int)cdiv(vocab, 256 * 8);
    if (nb < 1) nb = 1;
    if (nb > scratch_cap) nb = scratch_cap;
    const size_t off = (size_t)(rows - 1) * vocab;
    if (dtype == 0) argmax_stage1<float><<<nb, 256, 0, s>>>((const float*)logits + off, vocab, scratch_val, scratch_idx);
    else argmax_stage1<bf16_t><<<nb, 256, 0, s>>>((const bf16_t*)logits + off, vocab, scratch_val, scratch_idx);
    argmax_stage2<<<1, 64, 0, s>>>(scratch_val, scratch_idx, nb, out);
}

// Greedy token of EVERY row (batched decode): the same two stages with the row in blockIdx.y; out[r] as si32.
template <typename T>
__global__ void argmax_rows_stage1(const T* __restrict__ logits, int64_t n, float* pv, int32_t* pi) {
    __shared__ float sv[4];
    __shared__ int32_t si[4];
    const T* row = logits + (int64_t)blockIdx.y * n;
    float best = -INFINITY;
    int32_t bidx = 0x7fffffff;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        const float v = ldf(row, i);
        if (v > best || (v == best && (int32_t)i < bidx)) { best = v; bidx = (int32_t)i; }
    }
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_down(best, off, 64);
        const int32_t oi = __shfl_down(bidx, off, 64);
        if (ov > best || (ov == best && oi < bidx)) { best = ov; bidx = oi; }
    }
    if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = best; si[threadIdx.x >> 6] = bidx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; ++w)
            if (sv[w] > best || (sv[w] == best && si[w] < bidx)) { best = sv[w]; bidx = si[w]; }
        pv[blockIdx.y * gridDim.x + blockIdx.x] = best;
        pi[blockIdx.y * gridDim.x + blockIdx.x] = bidx;
    }
}
__global__ void argmax_rows_stage2(const float* pv, const int32_t* pi, int nparts, int32_t* out) {
    float best = -INFINITY;
    int32_t bidx = 0x7fffffff;
    for (int i = threadIdx.x; i < nparts; i += 64) {
        const float v = pv[blockIdx.x * nparts + i];
        const int32_t id = pi[blockIdx.x * nparts + i];
        if (v > best || (v == best && id < bidx)) { best = v; bidx = id; }
    }
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_down(best, off, 64);
        const int32_t oi = __shfl_down(bidx, off, 64);
        if (ov > best || (ov == best && oi < bidx)) { best = ov; bidx = oi; }
    }
    if (threadIdx.x == 0) out[blockIdx.x] = bidx == 0x7fffffff ? 0 : bidx;
}
void argmax_rows(hipStream_t s, int dtype, const void* logits, int64_t rows, int64_t vocab, int32_t* out, float* scratch_val,
                 int32_t* scratch_idx, int scratch_cap) {
    if (rows <= 0) return;
    int nb = (int)cdiv(vocab, 256 * 8);
    if (nb > scratch_cap / (int)rows) nb = scratch_cap / (int)rows;
    if (nb < 1) nb = 1;
    const dim3 grid((unsigned)nb, (unsigned)rows);
    if (dtype == 0) argmax_rows_stage1<float><<<grid, 256, 0, s>>>((const float*)logits, vocab, scratch_val, scratch_idx);
    else argmax_rows_stage1<bf16_t><<<grid, 256, 0, s>>>((const bf16_t*)logits, vocab, scratch_val, scratch_idx);
    argmax_rows_stage2<<<(unsigned)rows, 64, 0, s>>>(scratch_val, scratch_idx, nb, out);
}

// The same two stages for callers that must not allocate: the per-block partial maxima (value, index) live in a
// file-scope device array instead of a buffer the backend allocated.  Each GPU holds its own copy of the array at its
// own address until the process ends; argmax_noalloc_init() resolves that address once per device (with the device
// current), and the launcher hands it to the kernels as an ordinary pointer argument.  Stage 1 overwrites every
// partial that stage 2 reads, so nothing has to start at zero; two calls that overlap on one GPU (two streams) race
// on the array.
constexpr int kNoAllocPartials = 4096;   // rows * blocks per row
static __device__ __align__(256) unsigned char scratch[kNoAllocPartials * (sizeof(float) + sizeof(int32_t))];
constexpr int kNoAllocMaxDevices = 64;
static void* g_noalloc_ptr[kNoAllocMaxDevices] = {};
static std::mutex g_noalloc_mu;

hipError_t argmax_noalloc_init(int device) {
    if (device < 0 || device >= kNoAllocMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> g(g_noalloc_mu);
    if (g_noalloc_ptr[device]) return hipSuccess;
    void* p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (!p) return hipErrorInvalidSymbol;
    // load the kernels' code now, so that the first call does not do it
    hipFuncAttributes fa{};
    (void)hipFuncGetAttributes(&fa, (const void*)argmax_rows_stage1<float>);
    (void)hipFuncGetAttributes(&fa, (const void*)argmax_rows_stage1<bf16_t>);
    (void)hipFuncGetAttributes(&fa, (const void*)argmax_rows_stage2);
    g_noalloc_ptr[device] = p;
    return hipSuccess;
}
int argmax_noalloc_max_rows() { return 64; }
bool argmax_rows_noalloc(hipStream_t s, int device, int dtype, const void* logits, int64_t rows, int64_t vocab, int32_t* out) {
    if (device < 0 || device >= kNoAllocMaxDevices || rows < 1 || rows > argmax_noalloc_max_rows()) return false;
    void* p = g_noalloc_ptr[device];   // the device address, never the array's name (a host-side stand-in)
    if (!p) return false;
    float* val = reinterpret_cast<float*>(p);
    int32_t* idx = reinterpret_cast<int32_t*>(reinterpret_cast<unsigned char*>(p) + kNoAllocPartials * sizeof(float));
    argmax_rows(s, dtype, logits, rows, vocab, out, val, idx, kNoAllocPartials);
    return true;
}

// Temperature sampling, single block: softmax(logits/T) then inverse CDF at u.  The running
// sum is taken in index order by one wave so the chosen token does not depend on launch shape.
// Temperature sampling as the reference's device path does it
// (crates/gpt-rs-backend-triton/src/kernels/sample_temperature_last_axis_f32.triton:24-72): Gumbel-max with a
// stateless per-index hash of (index ^ seed); the score of index i is logit_i / temperature - log(-log(u_i)), the
// token is the index of the largest score, the smallest index on ties.  seed = bits(random_u) * 747796405 +
// 2891336453 (runtime/sampling.rs:98-101).
__device__ __forceinline__ float gumbel_of(uint32_t idx, uint32_t seed) {
    uint32_t x = idx ^ seed;
    x ^= x >> 16;
    x *= 0x7FEB352Du;
    x ^= x >> 15;
    x *= 0x846CA68Bu;
    x ^= x >> 16;
    float u = ((float)x + 1.0f) * 2.3283064365386963e-10f;   // f32(1 / 4294967297) = 2^-32
    u = fmaxf(u, 1e-7f);
    u = fminf(u, 1.0f - 1e-7f);
    return -logf(-logf(u));
}
template <typename T>
__global__ void sample_temperature_kernel(const T* __restrict__ row, int64_t n, float inv_t, uint32_t seed, int64_t* out) {
    __shared__ float s_score[16];
    __shared__ int64_t s_idx[16];
    float best = -INFINITY;
    int64_t best_i = 0;
    for (int64_t i = threadIdx.x; i < n; i += blockDim.x) {
        const float sc = ldf(row, i) * inv_t + gumbel_of((uint32_t)i, seed);
        if (sc > best) { best = sc; best_i = i; }   // ascending i per thread: the first maximum stays
    }
    for (int off = 32; off > 0; off >>= 1) {
        const float os = __shfl_down(best, off, 64);
        const int64_t oi = __shfl_down(best_i, off, 64);
        if (os > best || (os == best && oi < best_i)) { best = os; best_i = oi; }
    }
    if ((threadIdx.x & 63) == 0) { s_score[threadIdx.x >> 6] = best; s_idx[threadIdx.x >> 6] = best_i; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < (int)(blockDim.x >> 6); ++w)
            if (s_score[w] > best || (s_score[w] == best && s_idx[w] < best_i)) { best = s_score[w]; best_i = s_idx[w]; }
        *out = best_i;
    }
}
void sample_temperature_last_row(hipStream_t s, int dtype, const void* logits, int64_t rows, int64_t vocab,
                                 float temperature, float u, int64_t* out) {
    const size_t off = (size_t)(rows - 1) * vocab;
    const float inv_t = 1.0f / temperature;
    uint32_t bits;
    memcpy(&bits, &u, 4);
    const uint32_t seed = bits * 747796405u + 2891336453u;
    if (dtype == 0) sample_temperature_kernel<float><<<1, 1024, 0, s>>>((const float*)logits + off, vocab, inv_t, seed, out);
    else sample_temperature_kernel<bf16_t><<<1, 1024, 0, s>>>((const bf16_t*)logits + off, vocab, inv_t, seed, out);
}

}  // namespace k
}  // namespace gptrs
