// MFMA tile GEMM for prefill-sized linear layers (M > 16): bf16 in / f32 accumulate / bf16 out on
// v_mfma_f32_32x32x16_bf16, and f32 throughout on v_mfma_f32_32x32x2_f32.
//
// Per lane the matrix cores want consecutive k of ONE row (A) or ONE column (B).  Activations x[M,K] are row-major,
// so A fragments are plain 16-byte loads.  Weights are stored [in,out] row-major (nn/layers/linear.rs:50-71), the
// wrong way round for B, so the GEMM reads a derived copy Wk[K/KPC][Npad][KPC] in which the KPC consecutive k of a
// column that fill 16 bytes (8 bf16 or 4 f32) are adjacent (Npad = N rounded up to the 128-column block tile, zero
// filled); the backend builds it once per weight and keeps it beside the original.  With it a block's B tile is, per
// 16-byte k-group, one contiguous 2 KiB run, and every data movement below is in 16-byte chunks whatever the type.
#include <algorithm>
#include <type_traits>

#include "kernels.hpp"
#include "device_utils.hpp"

namespace gptrs {
namespace k {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

// Element types of the GEMM: KPC = k per 16-byte chunk; mma() multiplies one 32 x (2 KPC) A fragment by one
// (2 KPC) x 32 B fragment (a lane holds the KPC values of its row / column in k-group lane / 32).
template <typename T> struct Mma;
template <> struct Mma<bf16_t> {
    static constexpr int KPC = 8;
    typedef bf16x8_t frag;
    static __device__ __forceinline__ f32x16_t mma(const frag& a, const frag& b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float ld(const bf16_t* p, int64_t i) { return bf16_to_f32(p[i]); }
    static __device__ __forceinline__ void st(bf16_t* p, int64_t i, float v) { p[i] = f32_to_bf16(v); }
};
template <> struct Mma<float> {
    static constexpr int KPC = 4;
    typedef f32x4_t frag;
    // four K = 2 products: element e of both fragments is k = 4 * (lane / 32) + e of the 8-k step
    static __device__ __forceinline__ f32x16_t mma(const frag& a, const frag& b, f32x16_t c) {
#pragma unroll
        for (int e = 0; e < 4; ++e) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], b[e], c, 0, 0, 0);
        return c;
    }
    static __device__ __forceinline__ float ld(const float* p, int64_t i) { return p[i]; }
    static __device__ __forceinline__ void st(float* p, int64_t i, float v) { p[i] = v; }
};

static inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

constexpr int kBN = 128;   // column padding unit of the derived weights
constexpr int kKb = 8;     // 16-byte k-groups per k tile: 64 k of bf16, 32 k of f32

static inline int kpc_of(int dtype) { return dtype == 0 ? 4 : 8; }
int64_t mfma_padded_n(int64_t n) { return cdiv(n, kBN) * kBN; }
size_t mfma_weight_bytes(int dtype, int64_t k, int64_t n) {
    return (size_t)cdiv(k, kpc_of(dtype)) * (size_t)mfma_padded_n(n) * 16;
}

// Wk[kb][n][i] = W[kb*KPC+i][n]; one thread per (kb, n); reads coalesced along n, one 16-byte store.
template <typename T>
__global__ __launch_bounds__(256) void k8_weights_kernel(const T* __restrict__ w, T* __restrict__ out, int64_t K, int64_t N,
                                                         int64_t Npad) {
    constexpr int KPC = Mma<T>::KPC;
    const int64_t n = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t kb = blockIdx.y;
    if (n >= Npad) return;
    alignas(16) T r[KPC];
#pragma unroll
    for (int i = 0; i < KPC; ++i) {
        const int64_t kx = kb * KPC + i;
        r[i] = (n < N && kx < K) ? w[kx * N + n] : T(0);
    }
    *reinterpret_cast<uint4*>(out + (kb * Npad + n) * KPC) = *reinterpret_cast<const uint4*>(r);
}

void mfma_pack_weights(hipStream_t s, int dtype, const void* w, void* out, int64_t k, int64_t n) {
    const int64_t npad = mfma_padded_n(n);
    dim3 grid((unsigned)cdiv(npad, 256), (unsigned)cdiv(k, kpc_of(dtype)));
    if (dtype == 0) k8_weights_kernel<float><<<grid, 256, 0, s>>>((const float*)w, (float*)out, k, n, npad);
    else k8_weights_kernel<bf16_t><<<grid, 256, 0, s>>>((const bf16_t*)w, (bf16_t*)out, k, n, npad);
}

// Weight-only quantised weights (bf16 activations): the GEMM reads the CODES, in the same k-grouped order, and turns
// them into the bf16 values of the dequantised matrix, bf16(code * scale), on the way into LDS; no dequantised copy
// exists.  Ck[kb][n] holds the 8 codes of k-group kb of column n with the sign bias added (int8: 8 bytes of q + 128;
// int4: one dword, nibble i = q(k = 8 kb + i) + 8), so a code converts with one unsigned-byte / bit-field instruction
// and one fma (u * s - bias * s is exactly (u - bias) * s, rounded once like the product the dequantiser forms).
// Padding (n >= N, k >= K) holds the code of zero.
template <int QF>
__global__ __launch_bounds__(256) void k8_codes_kernel(const uint8_t* __restrict__ q, uint32_t* __restrict__ out, int64_t K, int64_t N,
                                                       int64_t Npad) {
    const int64_t n = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t kb = blockIdx.y;
    if (n >= Npad) return;
    if (QF == 1) {
        uint32_t w[2] = {0x80808080u, 0x80808080u};
        if (n < N) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int64_t kx = kb * 8 + i;
                const uint32_t u = kx < K ? (uint32_t)(uint8_t)(q[kx * N + n] + 128u) : 128u;   // si8 [K, N]
                w[i >> 2] = (w[i >> 2] & ~(0xFFu << (8 * (i & 3)))) | (u << (8 * (i & 3)));
            }
        }
        *reinterpret_cast<uint2*>(out + (kb * Npad + n) * 2) = make_uint2(w[0], w[1]);
    } else {
        uint32_t w = 0x88888888u;
        if (n < N) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int64_t k2 = kb * 4 + j;   // ui8 [K / 2, N]: low nibble k = 2 k2, high nibble k = 2 k2 + 1
                const uint32_t b = 2 * k2 < K ? (uint32_t)(q[k2 * N + n] ^ 0x88u) : 0x88u;
                w = (w & ~(0xFFu << (8 * j))) | (b << (8 * j));
            }
        }
        out[kb * Npad + n] = w;
    }
}
size_t mfma_codes_bytes(int64_t k, int64_t n, int quant) {
    return (size_t)cdiv(k, 8) * (size_t)mfma_padded_n(n) * (quant == 1 ? 8 : 4);
}
void mfma_pack_codes(hipStream_t s, const void* q, void* out, int64_t k, int64_t n, int quant) {
    const int64_t npad = mfma_padded_n(n);
    dim3 grid((unsigned)cdiv(npad, 256), (unsigned)cdiv(k, 8));
    if (quant == 1) k8_codes_kernel<1><<<grid, 256, 0, s>>>((const uint8_t*)q, (uint32_t*)out, k, n, npad);
    else k8_codes_kernel<2><<<grid, 256, 0, s>>>((const uint8_t*)q, (uint32_t*)out, k, n, npad);
}
__device__ __forceinline__ uint32_t mfma_pack_bf16(float lo, float hi) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    f32x2_t f;
    f.x = lo; f.y = hi;
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));   // round to nearest even
}

__device__ __forceinline__ float mfma_finish(float v, float v2, bool dual, int act, float bias, bool has_res, float res) {
    if (dual) v = (v / (1.0f + expf(v * -1.0f))) * v2;        // activation.rs:141-162
    v += bias;                                                // tensor_ops.rs:42-56
    if (act == 1) v = (v * 0.5f) * (erff(v / 1.41421354f) + 1.0f);  // activation.rs:96-113
    if (has_res) v += res;
    return v;
}

// Block tile BM x BN (128x128 as launched), BK = 64, four waves in a 2x2 grid; each wave owns
// (BM/2) x (BN/2) outputs as TM x TN MFMA tiles of 32x32.  LDS holds two stages of fragments,
// k-group-major ([kb][row or column][8 k], one spare row per k-group as CK does on gfx950), so a
// fragment read is a contiguous 512 bytes per half-wave.  Per k tile: one barrier; the tile after
// next is fetched global -> registers while the current one is multiplied, and the registers are
// stored into the idle LDS stage in the middle of the multiply.  Fragment reads run one k-step
// (16 k) ahead of the MFMAs that consume them.
//
// The staging registers are native vectors and every load is unconditional (the index is clamped
// instead): with HIP's uint4 struct and a guarded load the compiler keeps the staging array in
// scratch memory and waits for every load at once, which cost a factor of four.
//
// Requires K % (8 KPC) == 0 (64 for bf16, 32 for f32); M and N are guarded (rows clamp on load, stores are masked; the derived
// weights are padded to whole 128-column tiles).
// DUAL: SwiGLU pair silu(x.W) * (x.W2).  The block covers BN/2 real columns; the B tile holds, per
// wave column, TN/2 fragments of W followed by the same columns of W2, so gate and up of one
// output meet in the same lane.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

// QF: 0 = wk / wk2 hold values; 1 / 2 = they hold int8 / int4 codes (see k8_codes_kernel) and `scale` / `scale2` the
// scale tensors of the two matrices ([N] per column, or [K / 128, N] per group of 128 k), T = bf16 only.
// KW: wave groups per workgroup.  With KW = 2 a workgroup has 8 waves: both groups of four own the same 2 x 2 layout of
// outputs, group g multiplies k-steps [2 g, 2 g + 2) of every tile, and the second group's accumulators reach the
// first through LDS before the epilogue.  A launch with fewer tiles than two per CU then still has 8 waves per CU to
// cover LDS and barrier waits (what two co-resident workgroups do for the launches with many tiles).
template <typename T, int BM, int BN, bool DUAL, int QF, int KW>
__global__ __launch_bounds__(256 * KW) void gemm_mfma_kernel(const T* __restrict__ x, const T* __restrict__ wk,
                                                        const T* __restrict__ wk2, const T* __restrict__ bias,
                                                        const T* __restrict__ residual, T* __restrict__ y,
                                                        int M, int K, int N, int Npad, int act, int NT, int MT,
                                                        const T* __restrict__ scale, const T* __restrict__ scale2,
                                                        int full_tiles, int splits, float* __restrict__ part,
                                                        unsigned* __restrict__ tickets, int out_f32) {
    constexpr int KPC = Mma<T>::KPC;
    constexpr int kBK = kKb * KPC;                            // k per tile
    typedef typename Mma<T>::frag frag_t;
    constexpr int SA = (BM + 1) * 16, SB = (BN + 1) * 16;     // bytes between k-groups
    constexpr int STAGE = kKb * (SA + SB);
    constexpr int TM = BM / 64, TN = BN / 64;
    constexpr int NTH = 256 * KW;
    constexpr int KSTEPS = kKb / 2 / KW;                      // k-steps (2 k-groups each) per wave and tile
    constexpr int CA = BM * kKb / NTH, CB = BN * kKb / NTH;   // 16-byte chunks per thread per tile
    static_assert(KW == 1 || (!DUAL && KSTEPS >= 1 && CA >= 1 && CB >= 1), "k-split layout");
    constexpr int WN = BN / 2;                                // B-tile columns per wave column
    constexpr int NREAL = DUAL ? BN / 2 : BN;                 // output columns per block
    static_assert(!DUAL || TN % 2 == 0, "dual tiles need an even number of column fragments");
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wg = wave >> 2;               // wave group
    const int wm = (wave >> 1) & 1, wn = wave & 1;
    // Tile order.  Consecutive workgroup ids go to the 8 XCDs in turn and each XCD has its own L2, so XCD c takes
    // the contiguous range [c * per, (c + 1) * per) of a grouped order in which up to 8 row blocks of one column
    // tile follow each other: the ~32 workgroups an XCD runs at a time then cover 8 row blocks x 4 column tiles, a
    // weight tile is fetched from memory once for all its row blocks (with row-major ids the 1024 column tiles of an
    // lm_head were each fetched once per row block) and an activation tile once per 4 column tiles.
    //
    // Tail split: tiles [full_tiles, total) of that order are the last, partly filled round of the launch; each is
    // taken by `splits` workgroups (ids behind the whole tiles' ids, so the XCDs share them) that multiply a contiguous
    // range of k tiles each and meet through `part` and a ticket per tile, see the end of the kernel.
    int bx, by;
    int t_begin = 0, t_end = K / kBK, tail = -1, split = 0;
    {
        const int total = NT * MT, per = (full_tiles + 7) / 8;
        int v;
        if (blockIdx.x < (unsigned)per * 8) {
            v = (int)(blockIdx.x % 8) * per + (int)(blockIdx.x / 8);
            if (v >= full_tiles) return;
        } else {
            const int u = (int)blockIdx.x - per * 8;
            tail = u / splits;
            split = u % splits;
            v = full_tiles + tail;
            if (v >= total) return;
            t_begin = (int)((int64_t)split * t_end / splits);
            t_end = (int)((int64_t)(split + 1) * t_end / splits);
        }
        const int gsz = 8 * NT, g = v / gsz, first = g * 8;
        const int gm = MT - first < 8 ? MT - first : 8;
        by = first + (v % gsz) % gm;
        bx = (v % gsz) / gm;
    }
    const int m0 = by * BM, n0 = bx * NREAL;

    // global -> LDS chunk assignment (16 bytes each)
    // A: chunk c -> kb = c % 8, row = c / 8: eight lanes read 128 contiguous bytes of one row
    // B: chunk c -> tile column = c % BN, kb = c / BN: contiguous runs of the k-grouped weights
    const T* a_src[CA];
    const T* b_src[CB];
    int a_dst[CA], b_dst[CB];
#pragma unroll
    for (int j = 0; j < CA; ++j) {
        const int c = tid + NTH * j;
        const int kb = c % kKb, row = c / kKb;
        int m = m0 + row;
        if (m > M - 1) m = M - 1;
        a_src[j] = x + (int64_t)m * K + kb * KPC;
        a_dst[j] = kb * SA + row * 16;
    }
#pragma unroll
    for (int j = 0; j < CB; ++j) {
        const int c = tid + NTH * j;
        const int bc = c % BN, bkb = c / BN;
        int col = n0 + bc;
        const T* src = wk;
        if (DUAL) {
            // tile column -> (wave column, gate|up, column inside the half)
            const int wcol = bc / WN, in_w = bc % WN, half = in_w / (WN / 2), cc = in_w % (WN / 2);
            col = n0 + wcol * (WN / 2) + cc;
            src = half ? wk2 : wk;
        }
        // codes: 8 (int8) or 4 (int4) bytes per k-group and column instead of 16
        constexpr int64_t CW = QF == 0 ? KPC * (int64_t)sizeof(T) : (QF == 1 ? 8 : 4);
        b_src[j] = reinterpret_cast<const T*>(reinterpret_cast<const unsigned char*>(src) + ((int64_t)bkb * Npad + col) * CW);
        b_dst[j] = kKb * SA + bkb * SB + bc * 16;
    }
    // quantised: every chunk of a thread belongs to ONE tile column (256 % BN == 0), so one scale per thread (int8) or
    // per thread and k tile (int4: a tile of 64 k lies inside one group of 128)
    const T* s_src = nullptr;
    float q_scale = 0.f, q_scale_next = 0.f;
    if (QF != 0) {
        static_assert(NTH % BN == 0, "one tile column per thread");
        const int bc = tid % BN;
        int col = n0 + bc;
        const T* sp = scale;
        if (DUAL) {
            const int wcol = bc / WN, in_w = bc % WN, half = in_w / (WN / 2), cc = in_w % (WN / 2);
            col = n0 + wcol * (WN / 2) + cc;
            sp = half ? scale2 : scale;
        }
        if (col > N - 1) col = N - 1;   // padding columns hold the code of zero
        s_src = sp + col;
        if (QF == 1) q_scale = Mma<T>::ld(s_src, 0);
    }

    f32x16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
    u32x4_t ra[CA], rb[QF == 0 ? CB : 1];
    u32x2_t rq8[QF == 1 ? CB : 1];
    uint32_t rq4[QF == 2 ? CB : 1];
    const int nt = t_end;
    // bytes between consecutive k tiles of Wk
    const int64_t b_tile_step = (int64_t)kKb * Npad * (QF == 0 ? KPC * (int64_t)sizeof(T) : (QF == 1 ? 8 : 4));
    auto gload = [&](int t, int part, int nparts) {
#pragma unroll
        for (int j = 0; j < CA; ++j)
            if (j % nparts == part) ra[j] = *reinterpret_cast<const u32x4_t*>(a_src[j] + (int64_t)t * kBK);
#pragma unroll
        for (int j = 0; j < CB; ++j) {
            if (j % nparts != part) continue;
            const unsigned char* p = reinterpret_cast<const unsigned char*>(b_src[j]) + (int64_t)t * b_tile_step;
            if (QF == 0) rb[j] = *reinterpret_cast<const u32x4_t*>(p);
            else if (QF == 1) rq8[j] = *reinterpret_cast<const u32x2_t*>(p);
            else rq4[j] = *reinterpret_cast<const uint32_t*>(p);
        }
        if (QF == 2 && part == nparts - 1) q_scale_next = Mma<T>::ld(s_src, (int64_t)(t * kBK / 128) * N);
    };
    // part p of NP: chunks j with j % NP == p
    auto lwrite = [&](int buf, int part, int nparts) {
        unsigned char* base = lds + buf * STAGE;
#pragma unroll
        for (int j = 0; j < CA; ++j)
            if (j % nparts == part) *reinterpret_cast<u32x4_t*>(base + a_dst[j]) = ra[j];
#pragma unroll
        for (int j = 0; j < CB; ++j) {
            if (j % nparts != part) continue;
            u32x4_t v;
            if (QF == 0) {
                v = rb[j];
            } else if (QF == 1) {
                const float nb = -128.0f * q_scale;
                const uint32_t a = rq8[j].x, b = rq8[j].y;
                v.x = mfma_pack_bf16(__builtin_fmaf((float)(a & 0xFFu), q_scale, nb), __builtin_fmaf((float)((a >> 8) & 0xFFu), q_scale, nb));
                v.y = mfma_pack_bf16(__builtin_fmaf((float)((a >> 16) & 0xFFu), q_scale, nb), __builtin_fmaf((float)(a >> 24), q_scale, nb));
                v.z = mfma_pack_bf16(__builtin_fmaf((float)(b & 0xFFu), q_scale, nb), __builtin_fmaf((float)((b >> 8) & 0xFFu), q_scale, nb));
                v.w = mfma_pack_bf16(__builtin_fmaf((float)((b >> 16) & 0xFFu), q_scale, nb), __builtin_fmaf((float)(b >> 24), q_scale, nb));
            } else {
                const float nb = -8.0f * q_scale;
                const uint32_t c = rq4[j];
                float f[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) f[i] = __builtin_fmaf((float)((c >> (4 * i)) & 0xFu), q_scale, nb);
                v.x = mfma_pack_bf16(f[0], f[1]);
                v.y = mfma_pack_bf16(f[2], f[3]);
                v.z = mfma_pack_bf16(f[4], f[5]);
                v.w = mfma_pack_bf16(f[6], f[7]);
            }
            *reinterpret_cast<u32x4_t*>(base + b_dst[j]) = v;
        }
    };
    const int a_rd = (wm * (BM / 2) + (lane & 31)) * 16 + (lane >> 5) * SA;
    const int b_rd = kKb * SA + (wn * WN + (lane & 31)) * 16 + (lane >> 5) * SB;
    frag_t af[2][TM], bfr[2][TN];
    auto fread = [&](int buf, int kk, int slot) {
        const unsigned char* base = lds + buf * STAGE;
#pragma unroll
        for (int i = 0; i < TM; ++i) af[slot][i] = *reinterpret_cast<const frag_t*>(base + a_rd + kk * 2 * SA + i * 32 * 16);
#pragma unroll
        for (int j = 0; j < TN; ++j) bfr[slot][j] = *reinterpret_cast<const frag_t*>(base + b_rd + kk * 2 * SB + j * 32 * 16);
    };

    gload(t_begin, 0, 1);
    if (QF == 2) q_scale = q_scale_next;
    lwrite(0, 0, 1);
    gload(t_begin + 1 < nt ? t_begin + 1 : t_begin, 0, 1);
    __syncthreads();
    fread(0, wg * KSTEPS, 0);
    // The order of issue inside a k-step is fixed by hand (the scheduling barriers): the fragments of the NEXT k-step
    // are requested before the MFMAs of this one, so their LDS latency runs under the matrix work; left to itself the
    // compiler sinks the reads below the MFMAs into the same registers and the matrix pipe waits for every fragment.
    // The tile's barrier sits between the two halves of the last k-step's MFMAs, and the first fragments of the next
    // tile are requested right behind it.
    // Unquantised operands: the stage index is a compile-time constant and the tile loop advances two tiles at a time, so
    // LDS addresses in the step loop are a register plus an immediate (vector additions beside MFMAs are not free: f32
    // M = 512, K = 3072, N = 768 63.8 -> 60.5 us).  With codes to convert the doubled loop body costs more than that
    // saves (int4: +4-8 %), so those keep the index in a register.
    auto tile_step = [&](auto stage, int t) {
        const int cur = stage;
#pragma unroll
        for (int kk = 0; kk < KSTEPS; ++kk) {
            if (kk + 1 < KSTEPS) fread(cur, wg * KSTEPS + kk + 1, (kk + 1) & 1);
            // tile t+1 goes registers -> LDS (codes are converted on the way) and tile t+2 memory -> registers a quarter
            // of the chunks per k-step, between the MFMAs; past the last tile this stores a copy nobody reads
            if (QF == 2 && kk == 0) q_scale = q_scale_next;   // the scale that came with tile t+1
            lwrite(cur ^ 1, kk, KSTEPS);
            gload(t + 2 < nt ? t + 2 : nt - 1, kk, KSTEPS);
            __builtin_amdgcn_sched_barrier(0);
            if (kk + 1 < KSTEPS) {
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        acc[i][j] = Mma<T>::mma(af[kk & 1][i], bfr[kk & 1][j], acc[i][j]);
            } else {
                static_assert(((KSTEPS - 1) & 1) == 1, "the last k-step's fragments are in slot 1, the next tile's first in slot 0");
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN / 2; ++j)
                        acc[i][j] = Mma<T>::mma(af[kk & 1][i], bfr[kk & 1][j], acc[i][j]);
                __builtin_amdgcn_sched_barrier(0);
                __syncthreads();
                fread(cur ^ 1, wg * KSTEPS, 0);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = TN / 2; j < TN; ++j)
                        acc[i][j] = Mma<T>::mma(af[kk & 1][i], bfr[kk & 1][j], acc[i][j]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    if constexpr (QF == 0) {
        int t = t_begin;
        for (; t + 2 <= nt; t += 2) {
            tile_step(std::integral_constant<int, 0>{}, t);
            tile_step(std::integral_constant<int, 1>{}, t + 1);
        }
        if (t < nt) tile_step(std::integral_constant<int, 0>{}, t);
    } else {
        for (int t = t_begin; t < nt; ++t) tile_step((t - t_begin) & 1, t);
    }

    if (KW == 2) {
        // the second wave group hands its sums over through LDS (the tiles in it are dead: the loop ended on a barrier)
        float* xch = reinterpret_cast<float*>(lds) + (wave & 3) * (TM * TN * 16 * 64);
        static_assert(KW == 1 || 4 * TM * TN * 16 * 64 * 4 <= 2 * STAGE, "exchange area fits the staging buffers");
        if (wg == 1) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int v = 0; v < 16; ++v) xch[((i * TN + j) * 16 + v) * 64 + lane] = acc[i][j][v];
        }
        __syncthreads();
        if (wg == 1) return;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] += xch[((i * TN + j) * 16 + v) * 64 + lane];
    }
    if (KW == 1 && tail >= 0) {
        // Partial sums of a split tile go to the workspace, [item][value][thread], through device-scope stores (coherent
        // across the L2s of the XCDs without cache maintenance); once they are acknowledged the workgroup draws the
        // tile's ticket.  The one that draws the last ticket adds all partials in split order, its own included, so
        // the result does not depend on which workgroup that is, leaves the ticket at zero and runs the epilogue.
        constexpr int E = TM * TN * 16;
        float* mine = part + ((int64_t)(tail * splits + split) * E) * 256 + tid;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    __hip_atomic_store(mine + ((i * TN + j) * 16 + v) * 256, acc[i][j][v], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __builtin_amdgcn_s_waitcnt(0x0F70);                         // vmcnt(0)
        asm volatile("" ::: "memory");
        unsigned* flag = reinterpret_cast<unsigned*>(lds);          // the tiles in LDS are dead (the loop ended on a barrier)
        __syncthreads();
        if (tid == 0) *flag = __hip_atomic_fetch_add(&tickets[tail], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (*flag != (unsigned)(splits - 1)) return;
        asm volatile("" ::: "memory");                              // the partials are read after the ticket is known
        if (tid == 0) __hip_atomic_store(&tickets[tail], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
        for (int q = 0; q < splits; ++q) {
            const float* src = part + ((int64_t)(tail * splits + q) * E) * 256 + tid;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        acc[i][j][v] += __hip_atomic_load(src + ((i * TN + j) * 16 + v) * 256, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    // epilogue: lane holds column (lane % 32), rows 8*(v/4) + 4*(lane/32) + v%4 of each 32x32 tile (passing the sums
    // through LDS to store rows of 8, as the LDS-direct kernel below does, changed nothing here: 19.0 against 19.1 us at
    // K = 192, M = 1024, N = 6144)
    constexpr int TNO = DUAL ? TN / 2 : TN;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TNO; ++j) {
            const int n = n0 + wn * (NREAL / 2) + j * 32 + (lane & 31);
            if (n >= N) continue;
            const float bv = bias ? Mma<T>::ld(bias, n) : 0.f;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int m = m0 + wm * (BM / 2) + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (m >= M) continue;
                // out_f32: the f32 accumulator (plus an f32 residual) is stored as it is
                const float r = residual ? (out_f32 ? reinterpret_cast<const float*>(residual)[(int64_t)m * N + n]
                                                    : Mma<T>::ld(residual, (int64_t)m * N + n)) : 0.f;
                const float g = acc[i][j][v];
                const float u = DUAL ? acc[i][DUAL ? j + TN / 2 : j][v] : 0.f;
                const float o = mfma_finish(g, u, DUAL, act, bv, residual != nullptr, r);
                if (out_f32) reinterpret_cast<float*>(y)[(int64_t)m * N + n] = o;
                else Mma<T>::st(y, (int64_t)m * N + n, o);
            }
        }
}

// ---------------------------------------------------------------------------------------------------------------
// bf16 GEMM whose tiles go memory -> LDS without passing through registers (global_load_lds_dwordx4), for unquantised
// bf16 operands.  Against the kernel above: no staging registers and no LDS store instructions, a ring of NST staged
// tiles (loads run NST - 1 tiles ahead), and tile shapes chosen per launch so that the tiles fill the 256 CUs in whole
// rounds (128 x 192 and 128 x 96 as well as 128 x 128).
//
// Workgroup: KW groups of WM x WN waves.  A wave owns 64 x (32 TN) outputs as 2 x TN fragments of 32 x 32; the tile is
// (64 WM) x (32 TN WN).  All groups share the staged tiles; group g multiplies k-steps [g KSW, (g + 1) KSW) of every
// tile (KSW = 4 / KW k-steps of 16) and the groups' sums meet through LDS before the epilogue, so a launch of one tile
// per CU still has 8 waves per CU.
//
// LDS, per stage: A as rows of 128 bytes (64 k), B k-group-major ([k-group][column][8 k]).  One load instruction moves
// 64 x 16 bytes to 1 KiB of consecutive LDS, lane l to byte 16 l, so the layout is fixed by WHICH 16 bytes of memory a
// lane asks for: in A, position p of row r holds k-group p ^ ((r >> 1) & 7); eight lanes still read one row's 128
// contiguous bytes, and a fragment read (32 rows x 2 k-groups) touches every bank once per 16 lanes.  B fragments are
// contiguous as they are.
//
// Order of issue, fixed by hand with scheduling barriers: the fragments of the next k-step are requested before the
// MFMAs of this one; in a tile's last k-step half the MFMAs are issued, then the wave waits for its own loads of the
// next tile (vmcnt, which counts only LDS-direct loads here), passes the barrier that makes that tile complete and this
// one free, requests the next tile's first fragments, issues the other half and, behind it, requests the tile NST
// ahead into the freed stage.  Loads past the last tile repeat it into a stage nobody reads, so the count the wait relies on never changes.
// DUAL (SwiGLU pair): the tile's first BN / 2 columns are columns of W, the others the same columns of W2.
// One load instruction: lane l asks for the 16 bytes at base + offset(l) (a scalar base and a 32-bit offset per lane, so
// stepping to the next k tile is scalar arithmetic; vector instructions in the step loop cost the matrix pipe issue
// slots: per-lane 64-bit addresses were 5-10 % slower) and they land at LDS byte lds_addr + 16 l.
__device__ __forceinline__ void gemm_lds_load16(unsigned voff, unsigned long long sbase, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(voff), "s"(sbase), "s"(lds_addr) : "memory", "m0");
}
__device__ __forceinline__ unsigned long long gemm_uniform64(unsigned long long p) {
    return ((unsigned long long)(unsigned)__builtin_amdgcn_readfirstlane((int)(p >> 32)) << 32) |
           (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)p);
}
template <int N> __device__ __forceinline__ void gemm_wait_loads() { asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory"); }

template <int NST, int WM, int WN, int TN, int KW, bool DUAL>
__global__ __launch_bounds__(64 * WM * WN * KW) void gemm_dma_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ wk,
                                                                   const bf16_t* __restrict__ wk2, const bf16_t* __restrict__ bias,
                                                                   const bf16_t* __restrict__ residual, bf16_t* __restrict__ y,
                                                                   int M, int K, int N, int Npad, int act, int NT, int MT, int out_f32,
                                                                   int splits, float* __restrict__ part, unsigned* __restrict__ tickets) {
    constexpr int BK = 64, KG = 8, ROWB = 128;
    constexpr int BM = 64 * WM, BN = 32 * TN * WN, NW = WM * WN * KW;
    constexpr int NREAL = DUAL ? BN / 2 : BN;                          // output columns per tile
    constexpr int A_BYTES = BM * ROWB, B_BYTES = BN * ROWB, STAGE = A_BYTES + B_BYTES;
    constexpr int LAI = A_BYTES / 1024, LBI = B_BYTES / 1024;          // load instructions per tile
    constexpr int LA = (LAI + NW - 1) / NW, LB = (LBI + NW - 1) / NW;  // per wave (a wave past the end repeats an earlier one)
    constexpr int LPT = LA + LB;
    constexpr int KSW = 4 / KW;
    static_assert(KSW == 2 || KSW == 4, "an even number of k-steps per wave and tile: the last one's fragments sit in slot 1");
    static_assert(!DUAL || WN == 2, "pair tiles: wave column 0 multiplies W, wave column 1 the same columns of W2");
    static_assert((NST - 2) * LPT < 64, "vmcnt is a 6-bit counter");
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wg = wave / (WM * WN), wq = wave % (WM * WN);
    const int wm = wq / WN, wn = wq % WN;
    int bx, by, tile, sidx;
    {
        // XCD c takes a contiguous range of a grouped tile order (see gemm_mfma_kernel)
        // splits > 1: `splits` neighbours of that order share a tile and take a contiguous range of its k tiles each
        const int total = NT * MT * splits, per = (total + 7) / 8;
        const int u = (int)(blockIdx.x % 8) * per + (int)(blockIdx.x / 8);
        if (u >= total) return;
        tile = u / splits;
        sidx = u % splits;
        const int v = tile;
        const int gsz = 8 * NT, g = v / gsz, first = g * 8;
        const int gm = MT - first < 8 ? MT - first : 8;
        by = first + (v % gsz) % gm;
        bx = (v % gsz) / gm;
    }
    const int m0 = by * BM, n0 = bx * NREAL;
    // what each of this wave's load instructions fetches (per lane) and where its KiB goes
    unsigned a_off[LA], b_off[LB];
    unsigned a_dst[LA], b_dst[LB];
#pragma unroll
    for (int j = 0; j < LA; ++j) {
        const int q = (wave * LA + j) % LAI;
        const int sl = q * 64 + lane, row = sl / KG, pos = sl % KG;
        int m = m0 + row;
        if (m > M - 1) m = M - 1;
        a_off[j] = (unsigned)((m - m0) * K * 2 + ((pos ^ ((row >> 1) & 7)) * 16));   // under 128 rows of K bf16: fits 32 bits (K < 2^23)
        a_dst[j] = q * 1024;
    }
    // DUAL: both matrices are addressed from the lower of the two pointers (the launcher has checked that the other
    // lies less than 2^32 bytes above it, a k tile included)
    const unsigned long long w_lo = DUAL && (unsigned long long)wk2 < (unsigned long long)wk ? (unsigned long long)wk2 : (unsigned long long)wk;
#pragma unroll
    for (int j = 0; j < LB; ++j) {
        const int q = (wave * LB + j) % LBI;
        const int sl = q * 64 + lane, kg = sl / BN, bc = sl % BN;
        int col = n0 + bc;
        unsigned long long src = (unsigned long long)wk;
        if (DUAL) {
            col = n0 + bc % NREAL;
            src = bc >= NREAL ? (unsigned long long)wk2 : (unsigned long long)wk;
        }
        if (col > Npad - 1) col = Npad - 1;
        b_off[j] = (unsigned)(src - w_lo) + (unsigned)(((unsigned long long)kg * Npad + col) * 16);
        b_dst[j] = A_BYTES + q * 1024;
    }
    const unsigned long long a_base = (unsigned long long)(x + (int64_t)m0 * K);
    const int64_t b_tile_step = (int64_t)KG * Npad * 16;
    const unsigned lds0 = (unsigned)(uintptr_t)lds;
    const int kt_all = K / BK, kt0 = (int)((int64_t)sidx * kt_all / splits);
    const int nt = (int)((int64_t)(sidx + 1) * kt_all / splits) - kt0;   // this workgroup's k tiles: [kt0, kt0 + nt)
    auto issue = [&](int t, int st) {
        if (t > nt - 1) t = nt - 1;
        t += kt0;
        const unsigned long long ab = gemm_uniform64(a_base + (unsigned long long)t * (BK * 2));
        const unsigned long long bb = gemm_uniform64(w_lo + (unsigned long long)(t * b_tile_step));
        const unsigned sbase = lds0 + st * STAGE;
#pragma unroll
        for (int j = 0; j < LA; ++j) gemm_lds_load16(a_off[j], ab, (unsigned)__builtin_amdgcn_readfirstlane((int)(sbase + a_dst[j])));
#pragma unroll
        for (int j = 0; j < LB; ++j) gemm_lds_load16(b_off[j], bb, (unsigned)__builtin_amdgcn_readfirstlane((int)(sbase + b_dst[j])));
    };
    f32x16_t acc[2][TN];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
    const int fsel = lane >> 5;
    const int b_rd = A_BYTES + (wn * 32 * TN + (lane & 31)) * 16;
    bf16x8_t af[2][2], bfr[2][TN];
    auto fread = [&](int st, int kk, int slot) {   // kk: k-step of the tile
        const unsigned char* base = lds + st * STAGE;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int row = wm * 64 + i * 32 + (lane & 31), kg = 2 * kk + fsel;
            af[slot][i] = *reinterpret_cast<const bf16x8_t*>(base + row * ROWB + ((kg ^ ((row >> 1) & 7)) * 16));
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) bfr[slot][j] = *reinterpret_cast<const bf16x8_t*>(base + b_rd + (2 * kk + fsel) * (BN * 16) + j * 512);
    };
    for (int st = 0; st < NST - 1; ++st) issue(st, st);
    gemm_wait_loads<(NST - 2) * LPT>();
    __syncthreads();
    issue(NST - 1, NST - 1);
    fread(0, wg * KSW, 0);
    // One k tile; the ring position is a compile-time constant (the tile loop below is unrolled over the ring), so every
    // LDS address of the step loop is a register plus an immediate: with the position in a register the six address
    // additions per tile cost 3 % on the 8-wave tiles and 8-10 % on the 4-wave ones.
    auto tile_step = [&](auto ring_pos, int t) {
        constexpr int ST = decltype(ring_pos)::value, ST1 = ST + 1 == NST ? 0 : ST + 1;
#pragma unroll
        for (int kk = 0; kk < KSW; ++kk) {
            if (kk + 1 < KSW) fread(ST, wg * KSW + kk + 1, (kk + 1) & 1);
            __builtin_amdgcn_sched_barrier(0);
            if (kk + 1 < KSW) {
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[kk & 1][i], bfr[kk & 1][j], acc[i][j], 0, 0, 0);
            } else {
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[0][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[kk & 1][0], bfr[kk & 1][j], acc[0][j], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                gemm_wait_loads<(NST - 2) * LPT>();
                __syncthreads();
                fread(ST1, wg * KSW, 0);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[1][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[kk & 1][1], bfr[kk & 1][j], acc[1][j], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                issue(t + NST, ST);   // behind the MFMAs: the address arithmetic and the requests run under them (6 % faster than ahead of them)
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    static_assert(NST == 3, "the tile loop is unrolled over a ring of three");
    {
        int t = 0;
        for (; t + 3 <= nt; t += 3) {
            tile_step(std::integral_constant<int, 0>{}, t);
            tile_step(std::integral_constant<int, 1>{}, t + 1);
            tile_step(std::integral_constant<int, 2>{}, t + 2);
        }
        if (t < nt) tile_step(std::integral_constant<int, 0>{}, t);
        if (t + 1 < nt) tile_step(std::integral_constant<int, 1>{}, t + 1);
    }
    gemm_wait_loads<0>();   // the repeated loads of the last tile have landed before LDS is used for anything else
    // The two k-groups swap halves through LDS (the staged tiles are dead behind the barrier): group g gives the sums of
    // fragment row 1 - g and keeps row g, so all 8 waves take part in the epilogue, 32 rows each.
    static_assert(KW == 2, "two k-groups");
    f32x16_t mine[TN];
    {
        float* give = reinterpret_cast<float*>(lds) + (wg * (WM * WN) + wq) * (TN * 16 * 64) + lane;
        const float* take = reinterpret_cast<const float*>(lds) + ((1 - wg) * (WM * WN) + wq) * (TN * 16 * 64) + lane;
        __syncthreads();
        if (wg == 0) {
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) give[(j * 16 + v) * 64] = acc[1][j][v];
        } else {
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) give[(j * 16 + v) * 64] = acc[0][j][v];
        }
        __syncthreads();
        if (wg == 0) {
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) mine[j][v] = acc[0][j][v] + take[(j * 16 + v) * 64];
        } else {
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) mine[j][v] = acc[1][j][v] + take[(j * 16 + v) * 64];
        }
        __syncthreads();   // every wave has taken its half before the area is written again
    }
    if (!DUAL && splits > 1) {
        // Split over k: the workgroups of a tile leave their sums in the workspace, [tile][split][wave][value][lane],
        // through device-scope stores (coherent across the XCDs' L2s without cache maintenance); once they are
        // acknowledged the workgroup draws the tile's ticket.  The one that draws the last ticket adds all partial sums
        // in split order, its own included, so the result does not depend on which workgroup that is, leaves the ticket
        // at zero and runs the epilogue.
        float* mine_at = part + ((int64_t)(tile * splits + sidx) * NW + wave) * (TN * 16 * 64) + lane;
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) __hip_atomic_store(mine_at + (j * 16 + v) * 64, mine[j][v], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __builtin_amdgcn_s_waitcnt(0x0F70);                         // vmcnt(0)
        asm volatile("" ::: "memory");
        unsigned* flag = reinterpret_cast<unsigned*>(lds);
        __syncthreads();
        if (tid == 0) *flag = __hip_atomic_fetch_add(&tickets[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        const unsigned drawn = *flag;
        __syncthreads();                                            // the flag has been read before its bytes are used again
        if (drawn != (unsigned)(splits - 1)) return;
        asm volatile("" ::: "memory");                              // the partial sums are read after the ticket is known
        if (tid == 0) __hip_atomic_store(&tickets[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) mine[j][v] = 0.f;
        for (int q = 0; q < splits; ++q) {
            const float* src = part + ((int64_t)(tile * splits + q) * NW + wave) * (TN * 16 * 64) + lane;
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) mine[j][v] += __hip_atomic_load(src + (j * 16 + v) * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    // Rows of 8 outputs: a wave's 32 x (32 TN) sums go through an LDS area of its own (a lane holds one column of
    // four-row groups, memory wants runs along a row); then bias, GELU and the residual are applied to 8 neighbours at a
    // time and leave in one 16-byte store (two for f32 results; element by element when N is not a multiple of 8).
    // DUAL: the wave columns are the two matrices (wn = 0: x.W, wn = 1: x.W2, same output columns), so the pair of
    // waves meets here: each takes half of the pair's chunks and reads both areas.
    constexpr int RSF = 32 * TN + 4;     // floats per row of an area
    constexpr int CH = 32 * TN / 8;      // chunks of 8 per row
    constexpr int PASSES = 32 * CH / 64 / (DUAL ? 2 : 1);
    static_assert((32 * CH) % (DUAL ? 128 : 64) == 0, "whole passes of the wave");
    {
        float* tr = reinterpret_cast<float*>(lds) + wave * (32 * RSF);
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) tr[(8 * (v >> 2) + 4 * (lane >> 5) + (v & 3)) * RSF + j * 32 + (lane & 31)] = mine[j][v];
    }
    if (DUAL) __syncthreads();
    const float* area = reinterpret_cast<const float*>(lds) + (DUAL ? wave - wn : wave) * (32 * RSF);
    const int mrow0 = m0 + wm * 64 + wg * 32, ncol0 = DUAL ? n0 : n0 + wn * 32 * TN;
    const bool vec = (N & 7) == 0;
#pragma unroll
    for (int it = 0; it < PASSES; ++it) {
        const int c = (DUAL ? wn * PASSES + it : it) * 64 + lane, r = c / CH, cc = c % CH;
        const int m = mrow0 + r, n = ncol0 + cc * 8;
        if (m >= M || n >= N) continue;
        float o[8];
        *reinterpret_cast<f32x4_t*>(o) = *reinterpret_cast<const f32x4_t*>(area + r * RSF + cc * 8);
        *reinterpret_cast<f32x4_t*>(o + 4) = *reinterpret_cast<const f32x4_t*>(area + r * RSF + cc * 8 + 4);
        if (DUAL) {
            float u[8];
            *reinterpret_cast<f32x4_t*>(u) = *reinterpret_cast<const f32x4_t*>(area + 32 * RSF + r * RSF + cc * 8);
            *reinterpret_cast<f32x4_t*>(u + 4) = *reinterpret_cast<const f32x4_t*>(area + 32 * RSF + r * RSF + cc * 8 + 4);
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = (o[e] / (1.0f + expf(o[e] * -1.0f))) * u[e];   // activation.rs:141-162
        }
        const int64_t at = (int64_t)m * N + n;
        if (vec) {
            if (bias) {
                const u32x4_t bw = *reinterpret_cast<const u32x4_t*>(bias + n);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    o[2 * e] += __uint_as_float(bw[e] << 16);            // tensor_ops.rs:42-56
                    o[2 * e + 1] += __uint_as_float(bw[e] & 0xFFFF0000u);
                }
            }
            if (act == 1) {
#pragma unroll
                for (int e = 0; e < 8; ++e) o[e] = (o[e] * 0.5f) * (erff(o[e] / 1.41421354f) + 1.0f);   // activation.rs:96-113
            }
            if (residual) {
                if (out_f32) {
                    const f32x4_t r0 = *reinterpret_cast<const f32x4_t*>(reinterpret_cast<const float*>(residual) + at);
                    const f32x4_t r1 = *reinterpret_cast<const f32x4_t*>(reinterpret_cast<const float*>(residual) + at + 4);
#pragma unroll
                    for (int e = 0; e < 4; ++e) { o[e] += r0[e]; o[4 + e] += r1[e]; }
                } else {
                    const u32x4_t rw = *reinterpret_cast<const u32x4_t*>(residual + at);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        o[2 * e] += __uint_as_float(rw[e] << 16);
                        o[2 * e + 1] += __uint_as_float(rw[e] & 0xFFFF0000u);
                    }
                }
            }
            if (out_f32) {
                *reinterpret_cast<f32x4_t*>(reinterpret_cast<float*>(y) + at) = *reinterpret_cast<const f32x4_t*>(o);
                *reinterpret_cast<f32x4_t*>(reinterpret_cast<float*>(y) + at + 4) = *reinterpret_cast<const f32x4_t*>(o + 4);
            } else {
                u32x4_t w;
#pragma unroll
                for (int e = 0; e < 4; ++e) w[e] = (uint32_t)f32_to_bf16(o[2 * e]) | ((uint32_t)f32_to_bf16(o[2 * e + 1]) << 16);
                *reinterpret_cast<u32x4_t*>(y + at) = w;
            }
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                if (n + e >= N) break;
                const float bv = bias ? bf16_to_f32(bias[n + e]) : 0.f;
                const float rv = residual ? (out_f32 ? reinterpret_cast<const float*>(residual)[at + e] : bf16_to_f32(residual[at + e])) : 0.f;
                const float f = mfma_finish(o[e], 0.f, false, act, bv, residual != nullptr, rv);
                if (out_f32) reinterpret_cast<float*>(y)[at + e] = f;
                else y[at + e] = f32_to_bf16(f);
            }
        }
    }
}

template <int NST, int WM, int WN, int TN, int KW, bool DUAL>
static void launch_dma(hipStream_t s, const MfmaLinearArgs& a, int splits = 1) {
    constexpr int BM = 64 * WM, BN = 32 * TN * WN, NREAL = DUAL ? BN / 2 : BN;
    constexpr int stage = (BM + BN) * 128, xch = WM * WN * KW * TN * 16 * 64 * 4, rows = WM * WN * KW * 32 * (32 * TN + 4) * 4;
    constexpr int lds_bytes = NST * stage > (xch > rows ? xch : rows) ? NST * stage : (xch > rows ? xch : rows);
    static_assert(lds_bytes <= 160 * 1024, "LDS of one CU");
    auto kern = gemm_dma_kernel<NST, WM, WN, TN, KW, DUAL>;
    static bool configured = false;
    if (!configured) {
        (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
        configured = true;
    }
    const int64_t nt = cdiv(a.n, NREAL), mt = cdiv(a.m, BM);
    if (splits > 1 && (DUAL || !a.part || !a.tickets || nt * mt > (int64_t)kSkinnyTickets ||
                       a.part_bytes < (size_t)(nt * mt) * splits * BM * BN * sizeof(float)))
        splits = 1;
    const unsigned grid = (unsigned)(cdiv(nt * mt * splits, 8) * 8);
    kern<<<grid, 64 * WM * WN * KW, lds_bytes, s>>>((const bf16_t*)a.x, (const bf16_t*)a.wk, (const bf16_t*)a.wk2, (const bf16_t*)a.bias,
                                                   (const bf16_t*)a.residual, (bf16_t*)a.y, (int)a.m, (int)a.k, (int)a.n,
                                                   (int)mfma_padded_n(a.n), a.act, (int)nt, (int)mt, a.out_f32, splits, (float*)a.part,
                                                   a.tickets);
}

// Which tiles an unquantised bf16 launch of the LDS-direct kernel takes: 128 x 192 (`wide`), 128 x 96, or 128 x 192 with
// every tile split two ways over k.  Estimated from what the kernels measure at M = 1024 (us): a round of wide tiles
// 8 + 0.72 per k tile, of narrow ones 7 + 0.45 (28 KB per k tile against 40 KB, for half the flops), of split wide ones
// 15 + 0.36 (half the k tiles; 7 us for 25 MB of partial sums out and in again).  N = 6144: 256 wide tiles; N = 3072:
// 256 narrow tiles at K = 4096 (36.7 us; split 38.5), 128 wide tiles split in two at K = 9216 (66.7 us; narrow 72.8);
// the 9216-wide pair: 768 tiles of 128 x 96 outputs.
struct DmaPlan { bool wide; int splits; };
static DmaPlan dma_plan(int64_t m, int64_t k, int64_t n) {
    const int64_t mt = cdiv(m, 128), kt = k / 64;
    const int64_t tw = mt * cdiv(n, 192), tn = mt * cdiv(n, 96);
    const double wide = (double)cdiv(tw, 256) * (8.0 + 0.72 * kt);
    const double narrow = (double)cdiv(tn, 256) * (7.0 + 0.45 * kt);
    static const bool allow_split = [] { const char* e = getenv("GPTRS_HIP_GEMM_TAILSPLIT"); return !(e && e[0] == '0'); }();
    const bool can_split = allow_split && kt >= 32 && tw <= (int64_t)kSkinnyTickets;
    const double split = can_split ? (double)cdiv(2 * tw, 256) * (15.0 + 0.36 * kt) : 1e30;
    if (split < wide && split < narrow) return {true, 2};
    return {wide <= narrow, 1};
}

bool mfma_gemm_supported(int dtype, int64_t m, int64_t k, int64_t n, int quant) {
    if (dtype != 0 && dtype != 2) return false;
    if (quant != 0 && (dtype != 2 || (quant == 2 && k % 128 != 0))) return false;
    const int64_t bk = kKb * kpc_of(dtype);
    return m > 16 && k >= bk && k % bk == 0 && n >= 1 && m < (1ll << 31) && n < (1ll << 31) - kBN && k < (1ll << 31) &&
           cdiv(m, 128) * cdiv(n, 64) < (1ll << 30);   // tile ids are ints
}

// Tail split of a launch of 128 x 128 tiles on a chip of 256 CUs: the tiles beyond the last multiple of 256 would run
// as a round of their own on a few CUs (576 pair tiles: 64 CUs work, 192 wait); split 2 or 4 ways over k they give
// every CU a share.  Returns the number of whole tiles; `splits` = 1 means no split.
static int64_t mfma_tail_plan(int64_t tiles, int64_t k_tiles, int* splits) {
    *splits = 1;
    static const bool allow = [] { const char* e = getenv("GPTRS_HIP_GEMM_TAILSPLIT"); return !(e && e[0] == '0'); }();
    const int64_t tail = tiles % 256;
    if (!allow || tiles <= 256 || tail == 0 || tail > 128 || tail > (int64_t)kSkinnyTickets) return tiles;
    int sp = tail <= 64 ? 4 : 2;
    while (sp > 1 && k_tiles < 4 * sp) sp /= 2;
    if (sp < 2) return tiles;
    *splits = sp;
    return tiles - tail;
}
// A launch of few 64 x 64 tiles (under a quarter of the CUs) splits EVERY tile over k between up to 16 workgroups, the
// same way (partial sums through the workspace, a ticket per tile, the last ticket adds them in split order): twelve
// tiles with 96 k-tiles each otherwise keep twelve CUs busy for 96 steps while 244 wait.  Returns the split (1: none).
static int mfma_few_tiles_split(int64_t tiles64, int64_t k_tiles) {
    static const bool allow = [] { const char* e = getenv("GPTRS_HIP_GEMM_TAILSPLIT"); return !(e && e[0] == '0'); }();
    if (!allow || tiles64 > 64 || tiles64 > (int64_t)kSkinnyTickets) return 1;
    int sp = 16;
    while (sp > 1 && (tiles64 * sp > 256 || k_tiles < 4 * sp)) sp /= 2;
    return sp;
}
size_t mfma_workspace_bytes(int dtype, int64_t m, int64_t k, int64_t n, bool dual, int quant) {
    if (!mfma_gemm_supported(dtype, m, k, n, quant)) return 0;
    const int64_t tiles = cdiv(m, 128) * cdiv(mfma_padded_n(n), dual ? 64 : 128);
    const int64_t k_tiles = k / (kKb * kpc_of(dtype));
    if (!dual && cdiv(m, 128) * cdiv(n, 128) < 128) {   // the 64 x 64 kernel runs (see mfma_gemm)
        const int64_t t64 = cdiv(m, 64) * cdiv(mfma_padded_n(n), 64);
        const int sp = mfma_few_tiles_split(t64, k_tiles);
        return sp > 1 ? (size_t)t64 * sp * 64 * 64 * sizeof(float) : 0;
    }
    int sp = 1;
    const int64_t full = mfma_tail_plan(tiles, k_tiles, &sp);
    size_t bytes = sp > 1 ? (size_t)(tiles - full) * sp * 128 * 128 * sizeof(float) : 0;
    if (dtype == 2 && quant == 0 && !dual) {   // the LDS-direct kernel may split its 128 x 192 tiles over k
        const DmaPlan p = dma_plan(m, k, n);
        if (p.wide && p.splits > 1) bytes = std::max(bytes, (size_t)(cdiv(m, 128) * cdiv(n, 192)) * p.splits * 128 * 192 * sizeof(float));
    }
    return bytes;
}

template <typename T, int BM, int BN, bool DUAL, int QF = 0, int KW = 1>
static void launch_mfma(hipStream_t s, const MfmaLinearArgs& a) {
    constexpr int lds_bytes = 2 * kKb * ((BM + 1) * 16 + (BN + 1) * 16);
    auto kern = gemm_mfma_kernel<T, BM, BN, DUAL, QF, KW>;
    static bool configured = false;  // the attribute is per function, not per stream or device state
    if (!configured) {
        (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
        configured = true;
    }
    const int64_t npad = mfma_padded_n(a.n);
    constexpr int nreal = DUAL ? BN / 2 : BN;
    const int64_t nt = cdiv(npad, nreal), mt = cdiv(a.m, BM);
    int64_t full = nt * mt;
    int splits = 1;
    if (KW == 1 && BM == 128 && BN == 128 && a.part && a.tickets) {
        int sp = 1;
        const int64_t f = mfma_tail_plan(nt * mt, a.k / (kKb * Mma<T>::KPC), &sp);
        if (sp > 1 && a.part_bytes >= (size_t)(nt * mt - f) * sp * BM * BN * sizeof(float)) { full = f; splits = sp; }
    }
    if (KW == 1 && BM == 64 && BN == 64 && !DUAL && a.part && a.tickets) {
        const int sp = mfma_few_tiles_split(nt * mt, a.k / (kKb * Mma<T>::KPC));
        if (sp > 1 && a.part_bytes >= (size_t)(nt * mt) * sp * BM * BN * sizeof(float)) { full = 0; splits = sp; }
    }
    const unsigned grid = (unsigned)(cdiv(full, 8) * 8 + (nt * mt - full) * splits);
    kern<<<grid, 256 * KW, lds_bytes, s>>>((const T*)a.x, (const T*)a.wk, (const T*)a.wk2, (const T*)a.bias, (const T*)a.residual, (T*)a.y,
                                      (int)a.m, (int)a.k, (int)a.n, (int)npad, a.act, (int)nt, (int)mt, (const T*)a.scale, (const T*)a.scale2,
                                      (int)full, splits, (float*)a.part, a.tickets, a.dtype == 2 ? a.out_f32 : 0);
}

void mfma_gemm(hipStream_t s, const MfmaLinearArgs& a) {
    // a problem with fewer 128 x 128 tiles than half the CUs runs on 64 x 64 tiles (four times the workgroups); one
    // with at most one tile per CU on 8-wave workgroups that split every tile's k-steps between two wave groups
    // (M = 1024, bf16: 192 tiles 46 -> 40 us at K = 4096 and 87 -> 72 us at K = 9216; 384 tiles 54 -> 56 us, not taken)
    const int64_t tiles = cdiv(a.m, 128) * cdiv(a.n, a.wk2 ? 64 : 128);
    const bool small = tiles < 128;
    static const bool allow_split = [] { const char* e = getenv("GPTRS_HIP_GEMM_KSPLIT"); return !(e && e[0] == '0'); }();
    const bool split = allow_split && !a.wk2 && !small && tiles <= 256;
    if (a.quant == 1) {
        if (a.wk2) launch_mfma<bf16_t, 128, 128, true, 1>(s, a);
        else if (small) launch_mfma<bf16_t, 64, 64, false, 1>(s, a);
        else if (split) launch_mfma<bf16_t, 128, 128, false, 1, 2>(s, a);
        else launch_mfma<bf16_t, 128, 128, false, 1>(s, a);
    } else if (a.quant == 2) {
        if (a.wk2) launch_mfma<bf16_t, 128, 128, true, 2>(s, a);
        else if (small) launch_mfma<bf16_t, 64, 64, false, 2>(s, a);
        else if (split) launch_mfma<bf16_t, 128, 128, false, 2, 2>(s, a);
        else launch_mfma<bf16_t, 128, 128, false, 2>(s, a);
    } else if (a.dtype == 0) {
        if (a.wk2) launch_mfma<float, 128, 128, true>(s, a);
        else if (small) launch_mfma<float, 64, 64, false>(s, a);
        else if (split) launch_mfma<float, 128, 128, false, 0, 2>(s, a);
        else launch_mfma<float, 128, 128, false>(s, a);
    } else {
        // unquantised bf16: the LDS-direct kernel, on the tiles dma_plan() picks
        const bool allow_dma = a.lds_direct != 0;
        // its loads address a k tile with 32-bit offsets from one scalar base: 128 rows of x, 8 k-groups of the padded
        // weights, and for a pair the distance between the two matrices
        const uint64_t w_span = (uint64_t)mfma_padded_n(a.n) * 128;
        const uint64_t w_dist = !a.wk2 ? 0 : (a.wk2 > a.wk ? (uint64_t)((const char*)a.wk2 - (const char*)a.wk) : (uint64_t)((const char*)a.wk - (const char*)a.wk2));
        const bool reach = a.k <= (1 << 22) && w_span < (1ull << 31) && w_dist + w_span < (1ull << 32);
        if (allow_dma && reach && !small && a.wk2) return launch_dma<3, 2, 2, 3, 2, true>(s, a);
        if (allow_dma && reach && !small) {
            const DmaPlan p = dma_plan(a.m, a.k, a.n);
            return p.wide ? launch_dma<3, 2, 2, 3, 2, false>(s, a, p.splits) : launch_dma<3, 2, 1, 3, 2, false>(s, a);
        }
        if (a.wk2) launch_mfma<bf16_t, 128, 128, true>(s, a);
        else if (small) launch_mfma<bf16_t, 64, 64, false>(s, a);
        else if (split) launch_mfma<bf16_t, 128, 128, false, 0, 2>(s, a);
        else launch_mfma<bf16_t, 128, 128, false>(s, a);
    }
}

}  // namespace k
}  // namespace gptrs
