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
