// Launchers for the HIP kernels (gfx950).  Plain-pointer interfaces; all launches are
// asynchronous on the given stream.  Shapes are validated by the executor before any call.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace gptrs {
namespace k {

constexpr int kMaxRank = 6;

// dst[dst_off + sum c_i*dst_stride_i] = src[src_off + sum c_i*src_stride_i] over `dims`.
// Strides in elements.  dyn: 0 static; 1 = add clamp(starts[i],0,dyn_max[i])*dyn_stride[i] to the
// SOURCE offset (DynamicSlice, cpu.rs:804-820); 2 = to the DEST offset (DynamicUpdateSlice).
struct CopyDesc {
    int rank = 0;
    int dyn = 0;
    int64_t total = 0;
    int64_t dst_off = 0, src_off = 0;
    int64_t dims[kMaxRank] = {};
    int64_t dst_stride[kMaxRank] = {};
    int64_t src_stride[kMaxRank] = {};
    int dyn_rank = 0;
    int64_t dyn_max[kMaxRank] = {};
    int64_t dyn_stride[kMaxRank] = {};
};
void copy_strided(hipStream_t s, void* dst, const void* src, int elem_size, const CopyDesc& d, const int32_t* starts);

// Up to 256 payload bytes travel as kernel arguments: an upload with no staging buffer and
// no host synchronisation (token ids, positions, update_starts, RoPE rows).
struct SmallPayload { uint32_t w[64]; };
void store_small(hipStream_t s, void* dst, const SmallPayload& p, int nbytes);
void fill_zero(hipStream_t s, void* dst, size_t nbytes);

// dtype: 0 f32, 2 bf16 (tags of include/gptrs_hip.h).  Math in f32, output rounded to dtype.
void unary(hipStream_t s, int dtype, int op, const void* x, void* y, int64_t n);
void binary(hipStream_t s, int dtype, int op, const void* a, const void* b, void* y, int64_t n);
// b is a scalar (broadcast literal) -- used when the rhs is BroadcastTo(scalar literal)
void binary_scalar(hipStream_t s, int dtype, int op, const void* a, float b, void* y, int64_t n);
void compare(hipStream_t s, int dtype, int op, const void* a, const void* b, uint8_t* y, int64_t n);
void select(hipStream_t s, int elem_size, const uint8_t* p, const void* t, const void* f, void* y, int64_t n);
void cast(hipStream_t s, int src_dtype, int dst_dtype, const void* x, void* y, int64_t n);
void iota(hipStream_t s, int32_t* y, int64_t outer, int64_t axis_len, int64_t inner);
// x viewed as [outer][axis_len][inner]; kind 0 sum 1 max 2 min; f32 accumulation
void reduce(hipStream_t s, int dtype, int kind, const void* x, void* y, int64_t outer, int64_t axis_len, int64_t inner);
// rows of `table` ([vocab][inner] elements of elem_size) by si32 index; an out-of-range index
// zero-fills the row and raises *err_flag (checked at the next synchronising call)
void take(hipStream_t s, int elem_size, const void* table, const int32_t* idx, void* y, int64_t n_idx,
          int64_t vocab, int64_t inner, int* err_flag);

// C[b][m][n] = sum_k A[b][m][k] * B[b][k][n]; element strides given per operand; f32 accumulate.
struct DotDesc {
    int64_t batch, m, n, k;
    int64_t a_sb, a_sm, a_sk;
    int64_t b_sb, b_sk, b_sn;
    int64_t c_sb, c_sm;  // C is [b][m][n] with n contiguous
};
// dtype: of A and B; out_f32: bf16 operands, the f32 accumulator is stored as f32 (DotGeneralSpec.out_dtype)
void dot_generic(hipStream_t s, int dtype, const void* a, const void* b, void* c, const DotDesc& d, bool out_f32 = false);

// last row of [rows][vocab] logits; ties -> smallest index; result (int64) written to *out
// greedy token of every row (rows * partial blocks <= scratch_cap), ties to the smallest index; out: si32[rows]
void argmax_rows(hipStream_t s, int dtype, const void* logits, int64_t rows, int64_t vocab, int32_t* out, float* scratch_val,
                 int32_t* scratch_idx, int scratch_cap);
void argmax_last_row(hipStream_t s, int dtype, const void* logits, int64_t rows, int64_t vocab, int64_t* out,
                     float* scratch_val, int32_t* scratch_idx, int scratch_cap);
// argmax_rows over a fixed device array of the library instead of caller scratch: no allocation anywhere.
// argmax_noalloc_init: once per device, with that device current (resolves the array's address on that GPU).
// argmax_rows_noalloc: false when the device was not initialised or rows is outside [1, argmax_noalloc_max_rows()].
hipError_t argmax_noalloc_init(int device);
int argmax_noalloc_max_rows();
bool argmax_rows_noalloc(hipStream_t s, int device, int dtype, const void* logits, int64_t rows, int64_t vocab, int32_t* out);
// temperature sampling with a caller-supplied uniform u (inverse-CDF over softmax(logits/T))
void sample_temperature_last_row(hipStream_t s, int dtype, const void* logits, int64_t rows, int64_t vocab,
                                 float temperature, float u, int64_t* out);

// ---- fused kernels (kernels_fused.hip) --------------------------------------------------
// y[r] = LN(x[r]) * gamma + beta over the last axis, two-pass (mean, then centred variance):
// ops/functional/normalization.rs:123-174.  inv_n is the f32-rounded 1/N multiplier.
void layer_norm(hipStream_t s, int dtype, const void* x, const void* gamma, const void* beta, void* y,
                int64_t rows, int64_t n, float inv_n, float eps);
// y = x * rsqrt(mean(x^2)+eps) * gamma: normalization.rs:183-217
void rms_norm(hipStream_t s, int dtype, const void* x, const void* gamma, void* y, int64_t rows, int64_t n,
              float inv_n, float eps);
// the same over f32 rows and gains with a bf16 result (the f32 value rounded once)
void rms_norm_f32_to_bf16(hipStream_t s, const void* x, const void* gamma, void* y, int64_t rows, int64_t n, float inv_n,
                          float eps);
void softmax_rows(hipStream_t s, int dtype, const void* x, void* y, int64_t rows, int64_t n);
void gelu(hipStream_t s, int dtype, const void* x, void* y, int64_t n, float half, float inv_div, float one);
void swiglu(hipStream_t s, int dtype, const void* gate, const void* up, void* y, int64_t n);  // up==nullptr: silu

// Linear layer y[M,N] = act(x[M,K] . W[K,N] + bias) (+ residual), W row-major [in,out]
// (nn/layers/linear.rs:50-71).  act: 0 none, 1 exact-erf gelu.  w2 != nullptr: SwiGLU pair,
// y = silu(x.W) * (x.W2).  Picks a bandwidth-bound GEMV kernel for small M and an MFMA tile
// kernel for large M.  `ws` is a scratch buffer of at least linear_workspace_bytes().
struct LinearArgs {
    int dtype;
    const void* x; const void* w; const void* w2; const void* bias; const void* residual;
    void* y;
    int64_t m, k, n;
    int act;
    void* ws; size_t ws_bytes;
    int* counters;  // >= kLinearCounters zero-initialised ints, left zero by every launch
};
constexpr int kLinearCounters = 4096;
size_t linear_workspace_bytes(int dtype, int64_t m, int64_t k, int64_t n, bool dual);
void linear(hipStream_t s, const LinearArgs& a);
// Decode GEMV (M <= 16) over a column-tiled copy of the weights, Wt[tile][k][v] with
// v = column % (16 bytes / element size): no split-K, one launch per linear layer.  gamma != nullptr
// fuses a preceding RMSNorm (x is then the un-normalised row; inv_n, eps as in rms_norm()).
struct TiledLinearArgs {
    int dtype;
    const void* x; const void* wt; const void* wt2; const void* gamma; const void* bias; const void* residual;
    void* y;
    int64_t m, k, n;
    int act;
    float inv_n, eps;
    const void* beta;   // with gamma: LayerNorm (normalization.rs:123-174) instead of RMSNorm
    // bf16 weights only.  out_f32: y and residual are f32 (the accumulator leaves unrounded).  x_f32 (with gamma, RMSNorm):
    // x and gamma are f32, the normalised row is rounded to bf16 once as it is staged.
    int out_f32 = 0, x_f32 = 0;
};
size_t tiled_weight_bytes(int dtype, int64_t k, int64_t n);
void tile_weights(hipStream_t s, int dtype, const void* w, void* wt, int64_t k, int64_t n);
bool gemv_tiled_supported(int dtype, int64_t m, int64_t k, int64_t n);
void gemv_tiled(hipStream_t s, const TiledLinearArgs& a);

// Batched-decode linear layers (2 <= M <= 16, bf16 or f32) on the matrix cores over a 16-column tiled, k-grouped copy
// of the weights, Ws[tile][K/KPC][16][KPC] with KPC = 8 (bf16) or 4 (f32) k per 16 bytes (kernels_skinny.hip).  ws2 != nullptr: SwiGLU pair.  act: 0 none, 1 gelu.
struct SkinnyLinearArgs {
    int dtype;   // 0 f32, 2 bf16
    const void* x; const void* ws; const void* ws2; const void* bias; const void* residual;
    void* y;
    int64_t m, k, n;
    int act;
    // split-K over workgroups (layers with few tiles): part = skinny_workspace_bytes() of scratch, tickets =
    // kSkinnyTickets counters zeroed once (every launch leaves them zero); without them the layer runs unsplit
    void* part; size_t part_bytes; unsigned* tickets;
    // weight-only quantised: quant 1 = int8 (scale [N]), 2 = int4 groups of 128 (scale [K/128, N]); ws / ws2 are then
    // the code copies of skinny_pack_codes, scale / scale2 the scale tensors as the program holds them (bf16)
    int quant; const void* scale; const void* scale2;
    int out_f32 = 0;   // bf16 only: y and residual are f32
};
bool skinny_quant_supported(int dtype, int64_t m, int64_t k, int64_t n, int qf);
size_t skinny_codes_bytes(int64_t k, int64_t n, int qf);
void skinny_pack_codes(hipStream_t s, const void* codes, void* out, int64_t k, int64_t n, int qf);
constexpr size_t kSkinnyTickets = 1024;
int skinny_ksplit(int64_t k, int64_t n);
size_t skinny_workspace_bytes(int64_t k, int64_t n, bool dual);
bool skinny_gemm_supported(int dtype, int64_t m, int64_t k, int64_t n);
size_t skinny_weight_bytes(int dtype, int64_t k, int64_t n);
void skinny_pack_weights(hipStream_t s, int dtype, const void* w, void* out, int64_t k, int64_t n);
void skinny_gemm(hipStream_t s, const SkinnyLinearArgs& a);

// ---- weight-only quantisation (kernels_quant.hip) ------------------------------------------
// Build-defined extension (the reference has no quantisation scheme, docs/backend.md:620-632):
//   int8: symmetric, one scale per output column of W[K,N]: s_n = bf16(max_k |W[k,n]| / 127) (1 when 0),
//         q = clamp(rint(W / s_n), -127, 127)
//   int4: symmetric, groups of 128 along K per column: s[g,n] = bf16(max |w| / 7) (1 when 0), q in [-7,7],
//         two per byte along K: byte[k/2, n] = (q[k] & 0xF) | ((q[k+1] & 0xF) << 4)
// All arithmetic in f32 with IEEE division and round-half-even, so the results are bit-identical to
// the numpy closed form.  dtype tags: 0 f32, 2 bf16 (of w / scales / dequantised output).
void quant_w8_scales(hipStream_t s, int dtype, const void* w, void* scales, int64_t k, int64_t n);
void quant_w8(hipStream_t s, int dtype, const void* w, const void* scales, int8_t* q, int64_t k, int64_t n);
void quant_w4g128_scales(hipStream_t s, int dtype, const void* w, void* scales, int64_t k, int64_t n);
void quant_w4g128(hipStream_t s, int dtype, const void* w, const void* scales, uint8_t* packed, int64_t k, int64_t n);
// out[k,n] = dtype(f32(q) * f32(scale))
void dequant_w8(hipStream_t s, int dtype, const int8_t* q, const void* scales, void* out, int64_t k, int64_t n);
void dequant_w4g128(hipStream_t s, int dtype, const uint8_t* packed, const void* scales, void* out, int64_t k, int64_t n);

// Persistent decode chain (kernels_chain.hip): a run of consecutive M = 1 bf16 linear layers in
// ONE launch of one workgroup per CU, phases separated by a grid barrier, weights read from a
// 4-column / k-pair tiled copy, Wc[tile][k/2][4][2].  `flags` of a phase: RMSNorm prologue
// (gamma, inv_n, eps), SwiGLU pair (weights of gate and up interleaved column by column in one
// copy), bias, exact-erf GELU, residual.  x, residual and y may be produced by earlier phases of
// the same launch.
constexpr int kChainCounters = 16;        // striped arrival counters of the grid barrier
constexpr int kChainMaxPhases = 192;
constexpr int kChainMaxXsWords = 12288;   // staged activation words (48 KiB): K <= 24576 for bf16 weights
constexpr size_t kChainBarrierBytes = (kChainCounters * 64 + 64) * sizeof(unsigned);  // zero-initialised once
// kChainOutF32: y and the residual are f32.  kChainXF32 (with kChainNorm): x and gamma are f32, the normalised row is
// rounded to bf16 once as it is staged.
// kChainLayerNorm (with kChainNorm, f32 phases only): LayerNorm with gains `gamma` and offsets `beta` instead of RMSNorm.
enum : int { kChainNorm = 1, kChainDual = 2, kChainGelu = 4, kChainResidual = 8, kChainBias = 16, kChainOutF32 = 32, kChainXF32 = 64,
             kChainLayerNorm = 128, kChainAttnFinal = 256 };
// weight format of a linear phase; kChainW32: f32 weights (16-byte word = 4 columns x 1 k) with f32 activations,
// bias, residual and output (the launch's attention phases then read f32 rows and caches as well)
enum : int { kChainW16 = 0, kChainW8 = 1, kChainW4 = 2, kChainW32 = 3 };
enum : int { kChainLinear = 0, kChainAttnPartial = 1, kChainAttnCombine = 2 };
// One phase of a chain.  Linear: y = act(norm?(x) . W + bias) (+ residual).  Decode attention
// (attention.rs:657-779, T = 1) takes two phases: "partial" appends this step's K/V row and leaves
// one online-softmax record (max, sum, weighted V) per query head and position chunk in `part`;
// "combine" merges the records of a head into the context row y.
struct ChainPhase {
    int kind, flags;
    const void* w; const void* x; const void* gamma; const void* bias; const void* residual;
    void* y;
    int K, N, Kw, ntiles, wpt, units, upb, lds_bytes;
    float inv_n, eps;
    // quantised weights: wfmt 1 = int8 (16-byte word = 4 columns x 4 k, biased by 128; `scale`/`scale2` = the
    // per-column scale tensors of W and of the SwiGLU partner, as wscale/wscale2), wfmt 2 = int4 groups of 128 (word = 4 columns x 8 k,
    // biased by 8; `wscale` = derived copy sc[tile][group][4] bf16, staged into LDS behind the activations)
    int wfmt, lds_total;   // lds_total: lds_bytes plus what the phase stages behind the activations
    const void* wscale; const void* wscale2;
    // attention: x = packed qkv row [(n_q + 2 n_kv) * head_dim], y = context row [n_q * head_dim]
    void* k_cache; void* v_cache;              // [n_kv, capacity, head_dim], updated in place
    const int32_t* update_starts;              // si32[3]
    const int32_t* query_start;                // si32[1]
    const void* cos; const void* sin;          // RoPE rows of this position, or null (qkv already rotated)
    float* part;                               // [n_q][nch][head_dim + 2] f32
    int n_q, n_kv, head_dim, capacity, rot_half, nch;
    float scale;
    int pad;
    const void* beta;                          // LayerNorm offsets (kChainLayerNorm)
};
int chain_grid();  // workgroups per launch (one per CU), 0 when no device is current
bool chain_supported(int dtype, int64_t m, int64_t k, int64_t n, bool dual, bool norm, int wfmt = kChainW16, bool x_f32 = false, bool plain = false);
size_t chain_weight_bytes(int64_t k, int64_t n, bool dual, int wfmt = kChainW16);
// w2 != nullptr: SwiGLU pair, columns of w (gate) and w2 (up) interleaved.  wfmt 0: w is bf16 [k,n];
// 1: si8 [k,n]; 2: packed int4, ui8 [k/2,n]; 3: f32 [k,n] (no pair)
void chain_pack_weights(hipStream_t s, const void* w, const void* w2, void* out, int64_t k, int64_t n, int wfmt = kChainW16);
// bf16 copies only: the row-major matrix (of a pair: whichever of w / w2 is non-null) back out of the packed copy, exactly
void chain_unpack_weights(hipStream_t s, const void* packed, void* w, void* w2, int64_t k, int64_t n, bool dual);
// int4 only: derived scale copy sc[tile][group][4] (bf16) from s [k/128, n] (and the partner's s2)
size_t chain_scale_bytes(int64_t k, int64_t n, bool dual);
void chain_pack_scales_w4(hipStream_t s, int dtype, const void* sc, const void* sc2, void* out, int64_t k, int64_t n);
// fills K, N, Kw, ntiles, wpt, units, upb, lds_bytes, wfmt (and the dual flag); false when one workgroup would
// own more bias/residual columns than the kernel stages
bool chain_fill_phase(ChainPhase& p, int64_t k, int64_t n, bool dual, int wfmt = kChainW16);
// Decode attention inside a chain: supported shapes, scratch for the per-chunk records, and the
// two phases (shape fields filled; the caller sets the pointers of both).
bool chain_attn_supported(int dtype, int64_t t, int64_t n_q, int64_t n_kv, int64_t head_dim, int64_t rot_half);
size_t chain_attn_part_bytes(int64_t n_q, int64_t n_kv, int64_t head_dim);
// phases a decode attention takes: 2, or 1 for a cache of at most 128 positions (one chunk per kv head; the "partial"
// phase then writes the context row itself, kChainAttnFinal, and `combine` is left untouched)
int chain_attn_phases(int64_t capacity);
void chain_fill_attn(ChainPhase& partial, ChainPhase& combine, int64_t n_q, int64_t n_kv, int64_t head_dim, int64_t capacity,
                     int64_t rot_half, float scale);
// bar: kChainBarrierBytes of device memory zeroed once; abort_flag: raised when a barrier wait
// gives up (every wave then leaves the kernel).  false: launch not possible (caller falls back).
// stall_phase >= 0 (tests of the give-up path): every workgroup expects one arrival too many at that phase's barrier.
bool chain_launch(hipStream_t s, const ChainPhase* dev_table, int nphases, int lds_bytes, unsigned* bar, int* abort_flag,
                  int wfmt = kChainW16, int stall_phase = -1);   // wfmt: the weight format of EVERY linear phase of the table

// Prefill GEMM (M > 16, bf16) on the matrix cores over a k-grouped copy of the weights,
// Wk8[K/8][Npad][8] (kernels_mfma.hip).  wk2 != nullptr: SwiGLU pair.
struct MfmaLinearArgs {
    int dtype;   // 0 f32, 2 bf16
    const void* x; const void* wk; const void* wk2; const void* bias; const void* residual;
    void* y;
    int64_t m, k, n;
    int act;
    // weight-only quantised (bf16 activations): quant 1 = int8 per column, 2 = int4 groups of 128; wk / wk2 are then
    // the k-grouped CODE copies (mfma_pack_codes) and scale / scale2 the matrices' scale tensors
    int quant;
    const void* scale; const void* scale2;
    // tail split: when the last round of 128 x 128 tiles would leave most CUs idle, those tiles are split over k between
    // 2 or 4 workgroups that meet through `part` (mfma_workspace_bytes() of scratch) and `tickets` (kSkinnyTickets
    // counters, zero before and after every launch); without them every tile runs whole
    void* part = nullptr; size_t part_bytes = 0; unsigned* tickets = nullptr;
    int out_f32 = 0;   // bf16 only: y and residual are f32
    int lds_direct = 1;   // unquantised bf16: the LDS-direct kernel where it applies (0: the register-staged one)
};
size_t mfma_workspace_bytes(int dtype, int64_t m, int64_t k, int64_t n, bool dual, int quant);
size_t mfma_weight_bytes(int dtype, int64_t k, int64_t n);
void mfma_pack_weights(hipStream_t s, int dtype, const void* w, void* out, int64_t k, int64_t n);
size_t mfma_codes_bytes(int64_t k, int64_t n, int quant);
void mfma_pack_codes(hipStream_t s, const void* q, void* out, int64_t k, int64_t n, int quant);
bool mfma_gemm_supported(int dtype, int64_t m, int64_t k, int64_t n, int quant = 0);
void mfma_gemm(hipStream_t s, const MfmaLinearArgs& a);

// Rotate-half RoPE on packed [T, Q|K|V] rows (ops/functional/rotary.rs:430-536).
void rope_packed(hipStream_t s, int dtype, const void* qkv, const void* cos, const void* sin, void* out,
                 int64_t t, int64_t n_q, int64_t n_kv, int64_t head_dim, int64_t half);

// Decode attention over a fixed-capacity cache (ops/functional/attention.rs:657-779), T = 1.
// Appends this step's K/V rows at clamp(update_starts[1]) into k_out/v_out (which already hold
// the previous cache contents: either the donated buffers or a copy) and attends over positions
// 0..=query_start[0].
struct AttnDecodeArgs {
    int dtype;
    const void* qkv;            // [1, (n_q + 2 n_kv) * head_dim]
    void* k_cache; void* v_cache;  // [n_kv, capacity, head_dim], updated in place
    const int32_t* update_starts;  // si32[3]
    const int32_t* query_start;    // si32[1]
    void* ctx;                  // [1, n_q * head_dim]
    int64_t n_q, n_kv, head_dim, capacity;
    float scale;
    void* ws; size_t ws_bytes;
    // optional fused RoPE of Q and of the appended K row (qkv is then the pre-RoPE projection):
    // cos/sin rows [rot_half] of this position; requires rot_half % (16 / element size) == 0
    const void* cos; const void* sin; int64_t rot_half;
    // batch > 1: `batch` independent sequences in one launch: qkv is [batch, P], ctx [batch, n_q * head_dim], the caches
    // of sequence b are k_caches[b] / v_caches[b] (k_cache / v_cache are ignored), ws holds batch x the single size
    int batch;
    void* k_caches[16]; void* v_caches[16];
};
size_t attn_decode_workspace_bytes(int64_t n_q, int64_t head_dim, int64_t capacity);
int attn_decode(hipStream_t s, const AttnDecodeArgs& a);   // returns the number of launches it made

// Prefill causal attention (ops/functional/attention.rs:443-522): packed qkv [T, P] ->
// ctx [T, n_q*head_dim], and K/V in cache layout [n_kv, T, head_dim].
struct AttnPrefillArgs {
    int dtype;
    const void* qkv;
    void* ctx; void* k_out; void* v_out;
    int64_t t, n_q, n_kv, head_dim;
    float scale;
};
void attn_prefill(hipStream_t s, const AttnPrefillArgs& a);

// Causal attention over a growing cache (ops/functional/attention.rs:359-437, the `cache = Some` branch): T new rows of
// packed qkv [T, P] behind caches [n_kv, C, head_dim]: k_all / v_all [n_kv, C + T, head_dim] = the caches with the new
// rows appended, ctx [T, n_q*head_dim] = row i attends keys 0 .. C + i.  Two launches.
struct AttnConcatArgs {
    int dtype;
    const void* qkv; const void* k_cache; const void* v_cache;
    void* ctx; void* k_all; void* v_all;
    int64_t t, cache_len, n_q, n_kv, head_dim;
    float scale;
};
void attn_concat(hipStream_t s, const AttnConcatArgs& a);

}  // namespace k
}  // namespace gptrs
