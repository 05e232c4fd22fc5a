// Device helpers shared by the HIP kernels: bf16 <-> f32, wave64 reductions, 128-bit loads.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace gptrs {
namespace k {

typedef uint16_t bf16_t;  // raw bf16 bit pattern

__device__ __forceinline__ float bf16_to_f32(bf16_t v) { return __uint_as_float((uint32_t)v << 16); }
// round-to-nearest-even (docs/backend.md:99); NaN stays a quiet NaN
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (bf16_t)(u >> 16);
}
__device__ __forceinline__ float bf16lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    return (uint32_t)f32_to_bf16(lo) | ((uint32_t)f32_to_bf16(hi) << 16);
}

// Sum over the 64 lanes of a wave, result in every lane.  Cross-lane moves use DPP modifiers
// (register-to-register, VALU rate) instead of ds_bpermute: 16 x 6 bpermutes per thread at the end of
// a GEMV block kept the LDS pipe busy for ~4 us.  Steps: xor 1 and xor 2 inside quads, mirrored
// halves of 8 and 16 lanes, then lane 15 / lane 31 of the previous rows broadcast into rows 1,3 /
// 2,3; lane 63 then holds the total and is read back as a scalar.
__device__ __forceinline__ float wave_sum(float v) {
    int x = __float_as_int(v);
#define GPTRS_DPP_ADD(ctrl, row_mask)                                                                         \
    x = __float_as_int(__int_as_float(x) +                                                                     \
                       __int_as_float(__builtin_amdgcn_update_dpp(0, x, (ctrl), (row_mask), 0xf, false)))
    GPTRS_DPP_ADD(0xB1, 0xf);   // quad_perm [1,0,3,2]
    GPTRS_DPP_ADD(0x4E, 0xf);   // quad_perm [2,3,0,1]
    GPTRS_DPP_ADD(0x141, 0xf);  // row_half_mirror
    GPTRS_DPP_ADD(0x140, 0xf);  // row_mirror
    GPTRS_DPP_ADD(0x142, 0xa);  // row_bcast:15 into rows 1 and 3
    GPTRS_DPP_ADD(0x143, 0xc);  // row_bcast:31 into rows 2 and 3
#undef GPTRS_DPP_ADD
    return __int_as_float(__builtin_amdgcn_readlane(x, 63));
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

// Block-wide sum / max for blocks of up to 1024 threads (16 waves); every thread gets the result.
__device__ __forceinline__ float block_sum(float v, float* smem16) {
    v = wave_sum(v);
    const int w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) smem16[w] = v;
    __syncthreads();
    float r = 0.f;
    for (int i = 0; i < nw; ++i) r += smem16[i];
    return r;
}
__device__ __forceinline__ float block_max(float v, float* smem16) {
    v = wave_max(v);
    const int w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) smem16[w] = v;
    __syncthreads();
    float r = -INFINITY;
    for (int i = 0; i < nw; ++i) r = fmaxf(r, smem16[i]);
    return r;
}

}  // namespace k
}  // namespace gptrs
