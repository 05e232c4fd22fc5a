/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle helpers; never linked into or called by the
 * shipped HIP library.
 *
 * Plain-C restatement of the inner loops of the reference CPU interpreter
 * (crates/gpt-rs-backend-ref-cpu/src/cpu.rs) whose floating-point summation ORDER
 * matters for parity: every output element is accumulated sequentially over the
 * contraction / reduction index in f32, starting from 0 (or -inf / +inf).
 *
 * Build: gcc -O2 -fno-fast-math -ffp-contract=off (no FMA contraction, no
 * reassociation), so the k-outer loop nests below vectorise across outputs while
 * each output still sees exactly the reference's sequence of roundings.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

/* op_dot_general (cpu.rs:2196-2225): `sum += lhs[..]*rhs[..]` over the contraction
 * index, per (batch, lhs_free, rhs_free).  Operands arrive already permuted to
 * a[batch][m][k], b[batch][k][n] (the Python side does the axis bookkeeping). */
void oracle_bmm_f32(const float* a, const float* b, float* c,
                    size_t batch, size_t m, size_t k, size_t n) {
    for (size_t bi = 0; bi < batch; ++bi) {
        const float* ab = a + bi * m * k;
        const float* bb = b + bi * k * n;
        float* cb = c + bi * m * n;
        for (size_t i = 0; i < m; ++i) {
            float* crow = cb + i * n;
            for (size_t j = 0; j < n; ++j) crow[j] = 0.0f;
            for (size_t p = 0; p < k; ++p) {
                const float av = ab[i * k + p];
                const float* brow = bb + p * n;
                for (size_t j = 0; j < n; ++j) {
                    crow[j] = crow[j] + av * brow[j];
                }
            }
        }
    }
}

/* op_reduce (cpu.rs:1769-1790): x viewed as [outer][axis_len][inner]; kind 0=sum,
 * 1=max, 2=min.  Rust f32::max/min ignore a NaN operand, as fmaxf/fminf do. */
void oracle_reduce_f32(const float* x, float* y, size_t outer, size_t axis_len,
                       size_t inner, int kind) {
    for (size_t o = 0; o < outer; ++o) {
        for (size_t i = 0; i < inner; ++i) {
            const float* base = x + o * axis_len * inner + i;
            float acc = kind == 0 ? 0.0f : (kind == 1 ? -INFINITY : INFINITY);
            for (size_t a = 0; a < axis_len; ++a) {
                const float v = base[a * inner];
                acc = kind == 0 ? acc + v : (kind == 1 ? fmaxf(acc, v) : fminf(acc, v));
            }
            y[o * inner + i] = acc;
        }
    }
}

/* op_elementwise_unary (cpu.rs:1704-1714): libm single-precision routines.
 * op: 0 neg, 1 abs, 2 exp, 3 log, 4 tanh, 5 erf, 6 rsqrt (1/sqrt), 7 reciprocal. */
void oracle_unary_f32(const float* x, float* y, size_t n, int op) {
    for (size_t i = 0; i < n; ++i) {
        const float v = x[i];
        float r;
        switch (op) {
            case 0: r = -v; break;
            case 1: r = fabsf(v); break;
            case 2: r = expf(v); break;
            case 3: r = logf(v); break;
            case 4: r = tanhf(v); break;
            case 5: r = erff(v); break;
            case 6: r = 1.0f / sqrtf(v); break;
            default: r = 1.0f / v; break;
        }
        y[i] = r;
    }
}
