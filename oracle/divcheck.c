/* Exhaustive CPU proof obligation for the quantizer's fast quotient.
 *
 * TEST INFRASTRUCTURE (part of the CPU oracle; never linked into the product).
 *
 * The reference quantizers compute y = x / s with s = amax / 448 per group
 * (/root/reference/triton_kernels/deepseekv3/offical_kernel.py:14-15) or
 * s = (min(amax, 1e4) + 1e-8) / 448
 * (/root/reference/triton_kernels/dpsk_fp8linear/fp8.py:109-111).  The HIP
 * kernels replace the per-element IEEE division by one reciprocal per group and
 * a two-FMA correction:
 *
 *     r  = 1.0f / s                (correctly rounded, once per group)
 *     q0 = x * r
 *     e  = fmaf(q0, s, -x)         (exact negated residual)
 *     q  = fmaf(-e, r, q0)
 *
 * (the residual is kept negated so that x = -0 yields q = -0: with
 * e = fmaf(-q0, s, x) the two zero signs cancel to +0 and the sign bit of the
 * e4m3fn byte would be lost)
 *
 * x and amax are bfloat16, so there are only 2^15 possible amax values and 2^16
 * possible x: this program walks every pair with |x| <= amax, both dialects, and
 * counts where q differs from x / s as an fp32 pattern and as an e4m3fn byte.
 * It prints, per dialect, the set of amax biased exponents for which any e4m3fn
 * byte differs; the kernels take the plain-division path for exponents outside
 * the clean range that is hard-coded there, and the test asserts that range.
 *
 * Build: gcc -O2 -mfma -fopenmp -ffp-contract=off divcheck.c -o divcheck -lm
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static inline float bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static inline uint32_t f32_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

/* fp32 -> e4m3fn, round-to-nearest-even, non-saturating (overflow -> NaN). */
static uint8_t e4m3_encode(float f) {
    uint32_t u = f32_bits(f);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80);
    uint32_t mag = u & 0x7FFFFFFFu;
    if (mag >= 0x7F800000u) return sign | 0x7F;
    if (mag < 0x3C800000u) { /* below 2^-6: multiples of 2^-9 */
        double q = fabs((double)f) * 512.0;
        double r = nearbyint(q); /* default rounding mode: half-even */
        return sign | (uint8_t)r;
    }
    uint32_t lsb = (mag >> 20) & 1u;
    uint32_t rounded = (mag + 0x7FFFFu + lsb) & 0xFFF00000u;
    int e = (int)(rounded >> 23) - 127;
    int code = ((e + 7) << 3) | (int)((rounded >> 20) & 7u);
    if (code > 0x7E) return sign | 0x7F;
    return sign | (uint8_t)code;
}

static inline float sat448(float q) {
    if (q != q) return q;
    return q > 448.0f ? 448.0f : (q < -448.0f ? -448.0f : q);
}

int main(int argc, char** argv) {
    int verbose = argc > 1;
    int rc = 0;
    for (int mode = 0; mode < 2; ++mode) {
        long long n_pairs = 0, n_f32 = 0, n_fp8 = 0;
        long long fp8_by_exp[256];
        long long f32_by_exp[256];
        memset(fp8_by_exp, 0, sizeof fp8_by_exp);
        memset(f32_by_exp, 0, sizeof f32_by_exp);
#pragma omp parallel for schedule(dynamic, 64) reduction(+ : n_pairs, n_f32, n_fp8)
        for (int ai = 0; ai < 0x7F80; ++ai) { /* every finite non-negative bf16 amax */
            float amax = bf16_to_f32((uint16_t)ai);
            float s;
            if (mode == 0) {
                s = amax / 448.0f;
            } else {
                float c = amax > 1e4f ? 1e4f : amax;
                s = (c + 1e-8f) / 448.0f;
            }
            float r = 1.0f / s;
            long long lf32 = 0, lfp8 = 0;
            for (int xi = 0; xi <= ai; ++xi) {
                for (int sg = 0; sg < 2; ++sg) {
                    float x = bf16_to_f32((uint16_t)(xi | (sg << 15)));
                    float ref = x / s;
                    float q0 = x * r;
                    float e = fmaf(q0, s, -x);
                    __asm__ volatile("" : "+x"(e)); /* keep the compiler from folding the negation into the FMA above */
                    float q = fmaf(-e, r, q0);
                    uint8_t bref, bq;
                    if (mode == 0) {
                        bref = e4m3_encode(ref);
                        bq = e4m3_encode(q);
                    } else {
                        bref = e4m3_encode(sat448(ref));
                        bq = e4m3_encode(sat448(q));
                    }
                    /* NaN bytes compare equal whatever their sign */
                    int nan_both = ((bref & 0x7F) == 0x7F) && ((bq & 0x7F) == 0x7F);
                    if (f32_bits(ref) != f32_bits(q) && !(ref != ref && q != q)) ++lf32;
                    if (bref != bq && !nan_both) ++lfp8;
                    ++n_pairs;
                }
            }
            n_f32 += lf32;
            n_fp8 += lfp8;
            if (lf32 || lfp8) {
#pragma omp critical
                {
                    f32_by_exp[(ai >> 7) & 0xFF] += lf32;
                    fp8_by_exp[(ai >> 7) & 0xFF] += lfp8;
                }
            }
        }
        printf("mode %d pairs %lld f32_mismatch %lld fp8_mismatch %lld\n", mode, n_pairs, n_f32, n_fp8);
        int lo_clean = -1, hi_clean = -1, best_lo = -1, best_hi = -2;
        for (int e = 0; e < 255; ++e) {
            if (verbose && (f32_by_exp[e] || fp8_by_exp[e]))
                printf("  mode %d amax_exp %d f32 %lld fp8 %lld\n", mode, e, f32_by_exp[e], fp8_by_exp[e]);
            if (fp8_by_exp[e] == 0) {
                if (lo_clean < 0) lo_clean = e;
                hi_clean = e;
                if (hi_clean - lo_clean > best_hi - best_lo) {
                    best_lo = lo_clean;
                    best_hi = hi_clean;
                }
            } else {
                lo_clean = -1;
            }
        }
        printf("mode %d clean_amax_exp_range %d %d\n", mode, best_lo, best_hi);
    }
    return rc;
}
