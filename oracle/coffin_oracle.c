/*
 * CPU oracle for the quantized linear path of MuWinds/coffin.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the product package may link, load or
 * call this file; it exists so that tests, the smoke check and the CPU-baseline
 * leg of the benchmark have an independent, plain-C statement of what the
 * reference computes.  Every function names the reference lines it restates
 * (paths are relative to the reference tree).
 *
 * Pinning status (which independent check fixes each function) is listed in
 * oracle/README.md; functions without a pin are marked "parity unpinned" there.
 *
 * Build: make -C oracle   (gcc -O2 -fopenmp -ffp-contract=off)
 * -ffp-contract=off matters: every fused multiply-add below is spelled fmaf()
 * on purpose and every unfused product/sum must stay unfused.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ bf16 */

/* bf16 bit pattern -> fp32.  backends/corex/kernels/corex_scalar.h:31-34. */
static inline float bf16_to_f32(uint16_t v) {
    uint32_t u = ((uint32_t)v) << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* fp32 -> bf16, round to nearest even, finite inputs.
 * backends/corex/kernels/corex_scalar.h:37-41 (same rule as
 * backends/hip/kernels/gemv_int8.cu:35-39 and torch's .to(bfloat16)). */
static inline uint16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

void orc_bf16_from_f32(const float *src, uint16_t *dst, int64_t n) {
    for (int64_t i = 0; i < n; ++i) dst[i] = f32_to_bf16(src[i]);
}

void orc_bf16_to_f32(const uint16_t *src, float *dst, int64_t n) {
    for (int64_t i = 0; i < n; ++i) dst[i] = bf16_to_f32(src[i]);
}

int orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void orc_set_num_threads(int n) {
#ifdef _OPENMP
    omp_set_num_threads(n);
#else
    (void)n;
#endif
}

/* ------------------------------------------------- R0: QWeight.quantize */

/* Per-output-row symmetric absmax int8 quantisation of a dense [N,K] weight.
 * int8_weights.py:328-332:
 *   scale = w.abs().amax(-1).clamp_min(1e-8) / 127.0
 *   q     = (w / scale[:,None]).round().clamp_(-127,127).to(int8)
 * round() is round-half-even, the division is an IEEE fp32 division. */
void orc_qweight_quantize(const float *w, int64_t N, int64_t K, int8_t *wq,
                          float *scale) {
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n) {
        const float *row = w + n * K;
        float amax = 0.f;
        for (int64_t k = 0; k < K; ++k) amax = fmaxf(amax, fabsf(row[k]));
        const float s = fmaxf(amax, 1e-8f) / 127.0f;
        scale[n] = s;
        for (int64_t k = 0; k < K; ++k) {
            float q = rintf(row[k] / s);
            q = fminf(fmaxf(q, -127.f), 127.f);
            wq[n * K + k] = (int8_t)q;
        }
    }
}

/* QWeight.dequant to bf16: int8_weights.py:359
 *   (wq.float() * scale[:,None]).to(dtype)   -- one fp32 product, one narrowing
 * (tests/test_backends.py:889-903 pins the single rounding). */
void orc_qweight_dequant_bf16(const int8_t *wq, const float *scale, int64_t N,
                              int64_t K, uint16_t *dense) {
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n)
        for (int64_t k = 0; k < K; ++k)
            dense[n * K + k] = f32_to_bf16((float)wq[n * K + k] * scale[n]);
}

/* --------------------------------------- R3: per-token activation quant */

/* backends/reference/__init__.py:386-389 (_kv_quant):
 *   xf = x.float(); s = xf.abs().amax(-1).clamp_min(1e-5) / 127.0
 *   q  = (xf / s).round().clamp_(-127,127).to(int8)
 * x is bf16 (bit patterns).  IEEE division, round-half-even; the native
 * reciprocal form (backends/corex/kernels/w8a8.cu:99-103) is NOT what the
 * reference torch path computes and is not restated here. */
void orc_quant_act_i8(const uint16_t *x, int64_t M, int64_t K, int8_t *q,
                      float *s) {
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        const uint16_t *row = x + m * K;
        float amax = 0.f;
        for (int64_t k = 0; k < K; ++k) amax = fmaxf(amax, fabsf(bf16_to_f32(row[k])));
        const float sc = fmaxf(amax, 1e-5f) / 127.0f;
        s[m] = sc;
        for (int64_t k = 0; k < K; ++k) {
            float v = rintf(bf16_to_f32(row[k]) / sc);
            v = fminf(fmaxf(v, -127.f), 127.f);
            q[m * K + k] = (int8_t)v;
        }
    }
}

/* Proof obligation of the GPU quantiser, checked by exhaustion rather than by
 * argument.  The kernels do not divide per element: with r = 1.0f / sc (one IEEE
 * division per row) they form
 *     q0 = x * r;  e = fma(-q0, sc, x);  q1 = fma(e, r, q0)
 * and round q1 (by adding 1.5 * 2^23 and taking the low byte of the sum, unclamped).  This counts the (amax, x) pairs for which that differs from
 * rintf(x / sc) clamped to +-127 -- over every scale a row can have (amax = any
 * finite non-negative bf16 with bit pattern in [amax_lo, amax_hi)) and every
 * finite bf16 x with |x| <= amax.  With check_quotient != 0 the quotients
 * themselves must agree bit for bit wherever x / sc is a normal number.
 * Must return 0. */
int64_t orc_quant_division_mismatches(int32_t amax_lo, int32_t amax_hi, int32_t check_quotient) {
    int64_t bad = 0;
    if (amax_lo < 0) amax_lo = 0;
    if (amax_hi > 0x7F80) amax_hi = 0x7F80;
#pragma omp parallel for schedule(dynamic, 64) reduction(+ : bad)
    for (int32_t a = amax_lo; a < amax_hi; ++a) {
        const float amax = bf16_to_f32((uint16_t)a);
        const float sc = fmaxf(amax, 1e-5f) / 127.0f;
        const float r = 1.0f / sc;
        for (int32_t xb = 0; xb <= a; ++xb) {
            for (int sign = 0; sign < 2; ++sign) {
                const float x = bf16_to_f32((uint16_t)(xb | (sign << 15)));
                const float ref_q = x / sc;
                float ref = rintf(ref_q);
                ref = fminf(fmaxf(ref, -127.f), 127.f);
                const float q0 = x * r;
                const float e = fmaf(-q0, sc, x);
                const float q1 = fmaf(e, r, q0);
                /* the kernels round and narrow in one addition: q1 + 1.5 * 2^23 has a unit in the
                 * last place of 1, so the sum is q1 rounded to the nearest integer, ties to even, and
                 * its low byte is that integer in two's complement -- with no clamp, which is only
                 * right if the rounded value never leaves [-127, 127]; both are part of this check */
                const float magic = q1 + 12582912.0f;
                uint32_t mbits;
                memcpy(&mbits, &magic, 4);
                const int got = (int)(int8_t)(mbits & 0xffu);
                int differ = got != (int)ref || (mbits - 0x4B400000u + 127u) > 254u;
                if (check_quotient && fabsf(ref_q) >= 1.17549435e-38f) {
                    uint32_t u0, u1;
                    memcpy(&u0, &ref_q, 4);
                    memcpy(&u1, &q1, 4);
                    differ |= u0 != u1;
                }
                bad += differ;
            }
        }
    }
    return bad;
}

/* ------------------------------------------------ R7: W4 pack / unpack */

/* tools/quant_disk_w4a8.py:45-89 (quantize_projection), group_size along K:
 *   scale[g,n] = amax_{k in g}|w[n,k]|.clamp_min(1e-8) / 7.0
 *   q          = (w / scale).round().clamp_(-8,7)
 *   code       = q + 8;  byte[k/2, n] = code[2j] | code[2j+1] << 4
 * K is padded with zeros to a multiple of group_size (code 8) and then to an
 * even length.  packed is [ceil(Kpad/2), N] row-major, scale is [G, N]. */
void orc_w4_quantize(const float *w, int64_t N, int64_t K, int64_t gs,
                     uint8_t *packed, float *scale) {
    const int64_t G = (K + gs - 1) / gs;
    const int64_t Kp = G * gs;
    const int64_t Ke = (Kp + 1) / 2 * 2;
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n) {
        uint8_t *codes = (uint8_t *)malloc((size_t)Ke);
        for (int64_t k = 0; k < Ke; ++k) codes[k] = 8;
        for (int64_t g = 0; g < G; ++g) {
            float amax = 0.f;
            for (int64_t k = g * gs; k < (g + 1) * gs; ++k) {
                const float v = k < K ? w[n * K + k] : 0.f;
                amax = fmaxf(amax, fabsf(v));
            }
            const float s = fmaxf(amax, 1e-8f) / 7.0f;
            scale[g * N + n] = s;
            for (int64_t k = g * gs; k < (g + 1) * gs; ++k) {
                const float v = k < K ? w[n * K + k] : 0.f;
                float q = rintf(v / s);
                q = fminf(fmaxf(q, -8.f), 7.f);
                codes[k] = (uint8_t)((int)q + 8);
            }
        }
        for (int64_t j = 0; j < Ke / 2; ++j)
            packed[j * N + n] = (uint8_t)(codes[2 * j] | (codes[2 * j + 1] << 4));
        free(codes);
    }
}

static inline int w4_code(const uint8_t *packed, int64_t N, int64_t k, int64_t n) {
    const uint8_t b = packed[(k >> 1) * N + n];
    return (int)((b >> ((k & 1) * 4)) & 15) - 8;
}

/* tools/quant_disk_w4a8.py:118-128 (dequantize_projection) and
 * w4a8_weights.py:84-99 (W4A8Weight.rows/to): dense[n,k] = (nib-8)*scale[g,n],
 * fp32, [N,K]. */
void orc_w4_dequant_f32(const uint8_t *packed, const float *scale, int64_t N,
                        int64_t K, int64_t gs, float *dense) {
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n)
        for (int64_t k = 0; k < K; ++k)
            dense[n * K + k] = (float)w4_code(packed, N, k, n) * scale[(k / gs) * N + n];
}

/* --------------------------- R1 / R8: the reference torch linear (FP) */

/* backends/reference/__init__.py:93-95 with bf16 activations and a bf16
 * caps.weight_dtype: dense is rounded to bf16 once, the product runs on bf16
 * operands, the output is narrowed to bf16.  torch's CPU bf16 GEMM keeps an
 * fp32 accumulator in an unspecified order; this restatement accumulates in
 * double (k ascending) and narrows double -> fp32 -> bf16, which is inside any
 * order's rounding envelope.  Compared with a tolerance, never bit-wise.
 * dense: bf16 [N,K]; x: bf16 [M,K]; y: bf16 [M,N]. */
void orc_linear_bf16(const uint16_t *dense, const uint16_t *x, int64_t M, int64_t N,
                     int64_t K, uint16_t *y) {
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n) {
        for (int64_t m = 0; m < M; ++m) {
            double acc = 0.0;
            for (int64_t k = 0; k < K; ++k)
                acc += (double)bf16_to_f32(dense[n * K + k]) * (double)bf16_to_f32(x[m * K + k]);
            y[m * N + n] = f32_to_bf16((float)acc);
        }
    }
}

/* R1 in one call: QWeight -> bf16 dense -> linear.  Dequantises the whole
 * weight on every call exactly like reference._linear does. */
void orc_linear_qweight(const int8_t *wq, const float *scale, const uint16_t *x,
                        int64_t M, int64_t N, int64_t K, uint16_t *y) {
    uint16_t *dense = (uint16_t *)malloc((size_t)N * K * 2);
    orc_qweight_dequant_bf16(wq, scale, N, K, dense);
    orc_linear_bf16(dense, x, M, N, K, y);
    free(dense);
}

/* R8: W4A8Weight.to(bf16) then linear on UNQUANTISED activations
 * (backends/reference/__init__.py:94 via w4a8_weights.py:96-99). */
void orc_linear_w4weight(const uint8_t *packed, const float *scale, const uint16_t *x,
                         int64_t M, int64_t N, int64_t K, int64_t gs, uint16_t *y) {
    float *dense = (float *)malloc((size_t)N * K * 4);
    uint16_t *dense16 = (uint16_t *)malloc((size_t)N * K * 2);
    orc_w4_dequant_f32(packed, scale, N, K, gs, dense);
    orc_bf16_from_f32(dense, dense16, N * K);
    orc_linear_bf16(dense16, x, M, N, K, y);
    free(dense);
    free(dense16);
}

/* R2, the device meaning of "weight-only": the integer weight is NOT rounded
 * to bf16 first; y = bf16(scale[n] * sum_k wq[n,k]*x[m,k]) with the scale
 * applied once after the K-sum (backends/corex/kernels/gemv.cu:784-785,
 * :838-934; backends/hip/kernels/gemv_int8.cu:61-125).  Evaluated here in
 * double so it is the exact value any fp32 summation order approximates;
 * returns fp32 (not narrowed) so tests can measure a kernel's distance from
 * the exact answer.  yf: fp32 [M,N]. */
void orc_gemv_w8a16_exact(const int8_t *wq, const float *scale, const uint16_t *x,
                          int64_t M, int64_t N, int64_t K, float *yf) {
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n) {
        for (int64_t m = 0; m < M; ++m) {
            double acc = 0.0;
            for (int64_t k = 0; k < K; ++k)
                acc += (double)wq[n * K + k] * (double)bf16_to_f32(x[m * K + k]);
            yf[m * N + n] = (float)(acc * (double)scale[n]);
        }
    }
}

/* ----------------------------------------------------- R4: W8A8 GEMM */

/* acc[m,n] = sum_k xq[m,k]*wq[n,k] in int32, exact
 * (backends/corex/kernels/w8a8.cu:289-336); epilogue
 * y = bf16((float)acc * xs[m] * ws[n]), left to right, one narrowing
 * (w8a8.cu:208, w8a8_tcu.cu:297-298).  acc may be NULL.  y row stride ldy. */
void orc_gemm_w8a8(const int8_t *xq, const int8_t *wq, const float *xs, const float *ws,
                   int64_t M, int64_t N, int64_t K, int32_t *acc, uint16_t *y,
                   int64_t ldy) {
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        for (int64_t n = 0; n < N; ++n) {
            int32_t a = 0;
            const int8_t *xr = xq + m * K, *wr = wq + n * K;
            for (int64_t k = 0; k < K; ++k) a += (int32_t)xr[k] * (int32_t)wr[k];
            if (acc) acc[m * N + n] = a;
            if (y) {
                const float t = (float)a * xs[m];
                y[m * ldy + n] = f32_to_bf16(t * ws[n]);
            }
        }
    }
}

/* ------------------------------------------------ R5 / R6: W4A8 linear */

/* Per group g of gs consecutive k: sum_g = sum_k xq[m,k]*(nib(k,n)-8), int32
 * exact; total = fma((float)sum_g, ws[g,n], total) for g ascending from 0.f;
 * y = bf16(total * xs[m]).
 * backends/corex/kernels/w4a8.cu:56-195 (w4a8_dot with one split, w4a8_finish)
 * and backends/corex/kernels/w8a8_tcu.cu:484-499,561-573 (flush / final store).
 * The reference source writes `total += (float)sum * scale`; whether that
 * contracts to an fma is the reference compiler's choice and its GEMV kernel
 * additionally re-associates across 13..16 K-splits, so the reference itself
 * does not fix the fp32 association.  This oracle fixes it: one chain, groups
 * ascending, each step a single-rounding fma.  The int32 group sums are the
 * part the reference fixes exactly; group_acc ([M,G,N], may be NULL) exposes
 * them. */
void orc_linear_w4a8(const int8_t *xq, const float *xs, const uint8_t *packed,
                     const float *ws, int64_t M, int64_t N, int64_t K, int64_t gs,
                     int32_t *group_acc, uint16_t *y) {
    const int64_t G = (K + gs - 1) / gs;
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n) {
        int8_t *col = (int8_t *)malloc((size_t)K);
        for (int64_t k = 0; k < K; ++k) col[k] = (int8_t)w4_code(packed, N, k, n);
        for (int64_t m = 0; m < M; ++m) {
            float total = 0.f;
            for (int64_t g = 0; g < G; ++g) {
                const int64_t k1 = (g + 1) * gs < K ? (g + 1) * gs : K;
                int32_t sum = 0;
                for (int64_t k = g * gs; k < k1; ++k)
                    sum += (int32_t)xq[m * K + k] * (int32_t)col[k];
                if (group_acc) group_acc[(m * G + g) * N + n] = sum;
                total = fmaf((float)sum, ws[g * N + n], total);
            }
            if (y) y[m * N + n] = f32_to_bf16(total * xs[m]);
        }
        free(col);
    }
}

/* ------------------------------ fused producers of quantised activations */

/* exp(x) rounded once to fp32.  The reference evaluates silu in fp32 with its
 * library's expf (torch's vectorised routine, accurate to about one unit in the
 * last place, so the reference's own bits depend on the library); this oracle
 * fixes the ideal that routine approximates: the double-precision exp narrowed
 * once. */
static inline float expf_rounded_once(float x) { return (float)exp((double)x); }

/* silu(g) narrowed to bf16: g / (1 + exp(-g)), every operation in fp32.
 * backends/reference/__init__.py:253-268 (F.silu on a bf16 tensor computes in
 * fp32 and narrows); backends/corex/kernels/attn.cu:612-614. */
static inline uint16_t silu_bf16(uint16_t g_bits) {
    const float g = bf16_to_f32(g_bits);
    return f32_to_bf16(g / (1.f + expf_rounded_once(-g)));
}

void orc_silu_bf16(const uint16_t *g, uint16_t *out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = silu_bf16(g[i]);
}

/* Ops.silu_mul followed by Ops.kv_quant on its output, which is what
 * Ops.silu_mul_quant must equal bit for bit (backends/protocol.py:274-278,
 * backends/corex/kernels/attn.cu:594-641):
 *   s   = bf16(silu(gate))                    (first narrowing)
 *   out = bf16(float(s) * float(up))          (second narrowing; F.silu(gate) * up on bf16)
 *   q, sc = quant_act_i8(out)                 (absmax of the STORED bf16 values)
 * gate, up: bf16 [M,K] with row pitches ldg, ldu (elements); out bf16 [M,K] dense;
 * q int8 [M,K]; sc fp32 [M]. */
void orc_silu_mul_quant(const uint16_t *gate, const uint16_t *up, int64_t M, int64_t K,
                        int64_t ldg, int64_t ldu, uint16_t *out, int8_t *q, float *sc) {
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m)
        for (int64_t k = 0; k < K; ++k) {
            const float s = bf16_to_f32(silu_bf16(gate[m * ldg + k]));
            out[m * K + k] = f32_to_bf16(s * bf16_to_f32(up[m * ldu + k]));
        }
    if (q && sc) orc_quant_act_i8(out, M, K, q, sc);
}

/* Zero-centred RMSNorm of the reference, backends/reference/__init__.py:169-198:
 *   xf = x.float(); scale = rsqrt(mean(xf^2) + eps); y = (xf*scale).to(bf16) * w.to(bf16)
 * optionally after the residual add of :224-250 (x = bf16(x + add), written back).
 * The reference leaves the fp32 summation order of the mean to torch; this oracle
 * fixes the value every order approximates: the squares (exact in fp32: 8-bit
 * significands) are summed in double, k ascending -- exact, hence order-free,
 * whenever the row's magnitudes span less than 2^20 -- divided by N in double and
 * narrowed once.  rsqrt is 1/sqrt with both operations correctly rounded, as
 * torch's CPU kernel evaluates it.  The bf16 product of two bf16 tensors is one
 * fp32 multiply and one narrowing.
 * x: bf16 [M,N] with row pitch ldx, updated in place when add != NULL (pitch
 * lda); w: bf16 [N]; y: bf16 [M,N] dense. */
void orc_rms_norm(uint16_t *x, const uint16_t *add, const uint16_t *w, int64_t M, int64_t N,
                  int64_t ldx, int64_t lda, float eps, uint16_t *y) {
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        uint16_t *xr = x + m * ldx;
        if (add)
            for (int64_t k = 0; k < N; ++k)
                xr[k] = f32_to_bf16(bf16_to_f32(xr[k]) + bf16_to_f32(add[m * lda + k]));
        double ss = 0.0;
        for (int64_t k = 0; k < N; ++k) {
            const double v = (double)bf16_to_f32(xr[k]);
            ss += v * v;
        }
        const float ms = (float)(ss / (double)N);
        const float scale = 1.0f / sqrtf(ms + eps);
        for (int64_t k = 0; k < N; ++k) {
            const float normed = bf16_to_f32(f32_to_bf16(bf16_to_f32(xr[k]) * scale));
            y[m * N + k] = f32_to_bf16(normed * bf16_to_f32(w[k]));
        }
    }
}
