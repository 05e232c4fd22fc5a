/*
 * TEST INFRASTRUCTURE ONLY -- compiled into oracle/_ref/ (git-ignored) by oracle/Makefile.
 *
 * Drives the reference C backend's own matmul kernels, compiled from the reference checkout
 * where it lies (the #include directives below name files under $(REF_KERNELS); no reference
 * source is copied into this repository).  Concatenation order and the system headers follow
 * crates/gpt-rs-backend-c/src/kernels/mod.rs:1-16 and codegen/mod.rs:55-63.
 *
 * Used (a) to pin the oracle's dot_general against the reference's own arithmetic and (b) as
 * the timed CPU baseline (kind "reference") in bench.py.
 */
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>
#include <time.h>

#include "preamble.inc.c"
#if GPTRS_HAS_AVX512
#include "pack.inc.c"
#include "compute.inc.c"
#include "ukernel_16.inc.c"
#include "ukernel_32.inc.c"
#include "ukernel_48.inc.c"
#include "ukernel_64.inc.c"
#include "ukernel_misc.inc.c"
#endif
#include "api.inc.c"

int gptrs_ref_has_avx512(void) { return GPTRS_HAS_AVX512; }

/* gpt_rs_c_matmul_f32: C[m,n] = A[m,k] . B[k,n], no packed-B cache (api.inc.c). */
void gptrs_ref_matmul_f32(const float* a, const float* b, float* c, size_t m, size_t n, size_t k) {
    gpt_rs_c_matmul_f32(a, b, c, m, n, k);
}

/* One persistent packed-B cache per weight matrix, as the generated code keeps for dots whose rhs
 * is a program input (crates/gpt-rs-backend-c/src/codegen/emit/dot.rs:241-265). */
void* gptrs_ref_cache_new(void) { return calloc(1, sizeof(gpt_rs_bpack_cache)); }
void gptrs_ref_cache_free(void* p) {
    gpt_rs_bpack_cache* c = (gpt_rs_bpack_cache*)p;
    if (!c) return;
    if (c->bpack) gpt_rs_aligned_free(c->bpack);
    if (c->bpack32) gpt_rs_aligned_free(c->bpack32);
    if (c->bpack64) gpt_rs_aligned_free(c->bpack64);
    free(c);
}
void gptrs_ref_matmul_f32_cached(const float* a, const float* b, float* c, size_t m, size_t n, size_t k, void* cache) {
    gpt_rs_c_matmul_f32_cached_b(a, b, c, m, n, k, (gpt_rs_bpack_cache*)cache);
}
void gptrs_ref_matmul_f32_cached_bias(const float* a, const float* b, const float* bias, float* c, size_t m, size_t n,
                                      size_t k, void* cache) {
    gpt_rs_c_matmul_f32_cached_b_bias(a, b, bias, c, m, n, k, (gpt_rs_bpack_cache*)cache);
}

/* Timed loop for the CPU baseline: `iters` calls over `nmat` weight matrices (each with its own
 * warm packed-B cache), returning elapsed seconds.  x is [m,k], ws[i] is [k,n]. */
double gptrs_ref_time_matmuls(const float* x, const float* const* ws, void* const* caches, float* y, size_t nmat,
                              size_t m, size_t n, size_t k, int iters) {
    struct timespec t0, t1;
    for (size_t i = 0; i < nmat; ++i) gpt_rs_c_matmul_f32_cached_b(x, ws[i], y, m, n, k, (gpt_rs_bpack_cache*)caches[i]);
    clock_gettime(CLOCK_MONOTONIC, &t0);
    for (int it = 0; it < iters; ++it)
        for (size_t i = 0; i < nmat; ++i) gpt_rs_c_matmul_f32_cached_b(x, ws[i], y, m, n, k, (gpt_rs_bpack_cache*)caches[i]);
    clock_gettime(CLOCK_MONOTONIC, &t1);
    return (double)(t1.tv_sec - t0.tv_sec) + 1e-9 * (double)(t1.tv_nsec - t0.tv_nsec);
}

/*
 * GPT-2 decode step on the reference's kernels: every matrix product goes through
 * gpt_rs_c_matmul_f32_cached_b (m = 1: the packed-B GEMV path of compute.inc.c:662-713, cache warm); the other ops
 * are the plain loops the C backend's generated code runs for them (crates/gpt-rs-backend-c/src/codegen/emit/*.rs):
 * embedding add, two-pass LayerNorm, bias add, exact-erf GELU, attention over the valid cache rows with a max-shifted
 * softmax, residual adds, argmax.  Block wiring as crates/gpt-rs/src/model/gpt.rs:81-97, 585-751.
 * Weights in the order of GptRefWeights; kcache / vcache are [layers][heads][capacity][head_dim].
 */
typedef struct {
    const float* tok_emb; const float* pos_emb;           /* [V, d], [ctx, d] */
    const float* const* ln1_g; const float* const* ln1_b; /* per layer [d] */
    const float* const* w_qkv; const float* const* b_qkv; /* [d, 3d], [3d] */
    const float* const* w_out; const float* const* b_out; /* [d, d], [d] */
    const float* const* ln2_g; const float* const* ln2_b;
    const float* const* w_in; const float* const* b_in;   /* [d, f], [f] */
    const float* const* w_o2; const float* const* b_o2;   /* [f, d], [d] */
    const float* lnf_g; const float* lnf_b; const float* lm_head; /* [d], [d], [d, V] */
    void* const* caches;                                   /* 4 per layer + 1: packed-B caches */
    int layers, d, heads, f, vocab, capacity;
    float eps;
} GptRefWeights;

static void ref_layer_norm(const float* x, const float* g, const float* b, float* y, int n, float eps) {
    const float inv_n = 1.0f / (float)n;
    float s = 0.f;
    for (int i = 0; i < n; ++i) s += x[i];
    const float mean = s * inv_n;
    float q = 0.f;
    for (int i = 0; i < n; ++i) { const float c = x[i] - mean; q += c * c; }
    const float inv_std = 1.0f / sqrtf(q * inv_n + eps);
    for (int i = 0; i < n; ++i) y[i] = ((x[i] - mean) * inv_std) * g[i] + b[i];
}

/* scratch: 4 d + 3 d + f + capacity + vocab floats.  Returns the greedy token; logits_out may be NULL. */
int gptrs_ref_gpt2_decode_step(const GptRefWeights* W, int token, int pos, float* kcache, float* vcache, float* scratch,
                               float* logits_out) {
    const int d = W->d, H = W->heads, dh = d / H, f = W->f, C = W->capacity, V = W->vocab;
    float* x = scratch;            /* [d] residual stream */
    float* h = x + d;              /* [d] */
    float* ctx = h + d;            /* [d] */
    float* t = ctx + d;            /* [d] */
    float* qkv = t + d;            /* [3d] */
    float* ff = qkv + 3 * d;       /* [f] */
    float* sc = ff + f;            /* [capacity] */
    float* logits = logits_out ? logits_out : sc + C;
    const float scale = 1.0f / sqrtf((float)dh);
    for (int i = 0; i < d; ++i) x[i] = W->tok_emb[(size_t)token * d + i] + W->pos_emb[(size_t)pos * d + i];
    for (int l = 0; l < W->layers; ++l) {
        void* const* cc = W->caches + 4 * l;
        ref_layer_norm(x, W->ln1_g[l], W->ln1_b[l], h, d, W->eps);
        gpt_rs_c_matmul_f32_cached_b(h, W->w_qkv[l], qkv, 1, 3 * d, d, (gpt_rs_bpack_cache*)cc[0]);
        for (int i = 0; i < 3 * d; ++i) qkv[i] += W->b_qkv[l][i];
        float* K = kcache + (size_t)l * H * C * dh;
        float* Vc = vcache + (size_t)l * H * C * dh;
        for (int hd = 0; hd < H; ++hd) {
            memcpy(K + ((size_t)hd * C + pos) * dh, qkv + d + hd * dh, sizeof(float) * dh);
            memcpy(Vc + ((size_t)hd * C + pos) * dh, qkv + 2 * d + hd * dh, sizeof(float) * dh);
            const float* q = qkv + hd * dh;
            float mx = -INFINITY;
            for (int p = 0; p <= pos; ++p) {
                const float* kr = K + ((size_t)hd * C + p) * dh;
                float s = 0.f;
                for (int i = 0; i < dh; ++i) s += q[i] * kr[i];
                sc[p] = s * scale;
                if (sc[p] > mx) mx = sc[p];
            }
            float sum = 0.f;
            for (int p = 0; p <= pos; ++p) { sc[p] = expf(sc[p] - mx); sum += sc[p]; }
            float* o = ctx + hd * dh;
            for (int i = 0; i < dh; ++i) o[i] = 0.f;
            for (int p = 0; p <= pos; ++p) {
                const float w = sc[p] / sum;
                const float* vr = Vc + ((size_t)hd * C + p) * dh;
                for (int i = 0; i < dh; ++i) o[i] += w * vr[i];
            }
        }
        gpt_rs_c_matmul_f32_cached_b(ctx, W->w_out[l], t, 1, d, d, (gpt_rs_bpack_cache*)cc[1]);
        for (int i = 0; i < d; ++i) x[i] = (t[i] + W->b_out[l][i]) + x[i];
        ref_layer_norm(x, W->ln2_g[l], W->ln2_b[l], h, d, W->eps);
        gpt_rs_c_matmul_f32_cached_b(h, W->w_in[l], ff, 1, f, d, (gpt_rs_bpack_cache*)cc[2]);
        for (int i = 0; i < f; ++i) {
            const float v = ff[i] + W->b_in[l][i];
            ff[i] = (v * 0.5f) * (erff(v / 1.41421354f) + 1.0f);
        }
        gpt_rs_c_matmul_f32_cached_b(ff, W->w_o2[l], t, 1, d, f, (gpt_rs_bpack_cache*)cc[3]);
        for (int i = 0; i < d; ++i) x[i] = (t[i] + W->b_o2[l][i]) + x[i];
    }
    ref_layer_norm(x, W->lnf_g, W->lnf_b, h, d, W->eps);
    gpt_rs_c_matmul_f32_cached_b(h, W->lm_head, logits, 1, V, d, (gpt_rs_bpack_cache*)W->caches[4 * W->layers]);
    int best = 0;
    for (int i = 1; i < V; ++i) if (logits[i] > logits[best]) best = i;
    return best;
}

/* Greedy loop: feeds `prompt` one token at a time (positions 0 .. n_prompt - 1), then generates n_new tokens;
 * returns the seconds spent on the last n_timed steps (the steps before them are the warm-up). */
double gptrs_ref_gpt2_generate(const GptRefWeights* W, const int* prompt, int n_prompt, int n_new, int n_timed,
                               float* kcache, float* vcache, float* scratch, int* tokens_out) {
    struct timespec t0, t1;
    int tok = prompt[0], pos = 0;
    const int total = n_prompt + n_new - 1;   /* steps: the last generated token needs no forward */
    double elapsed = 0.0;
    for (int s = 0; s < total; ++s) {
        if (s == total - n_timed) clock_gettime(CLOCK_MONOTONIC, &t0);
        const int next = gptrs_ref_gpt2_decode_step(W, tok, pos, kcache, vcache, scratch, NULL);
        ++pos;
        if (s + 1 < n_prompt) tok = prompt[s + 1];
        else { tok = next; tokens_out[s + 1 - n_prompt] = next; }
    }
    clock_gettime(CLOCK_MONOTONIC, &t1);
    if (n_timed > 0 && n_timed <= total) elapsed = (double)(t1.tv_sec - t0.tv_sec) + 1e-9 * (double)(t1.tv_nsec - t0.tv_nsec);
    return elapsed;
}
