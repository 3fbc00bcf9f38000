/*
 * Exhaustive proof, on the CPU, of the short rounding sequence the fused quantisers use for rows
 * (columns) whose scale is a normal fp16 number.  There the scale comes from the data it divides,
 *     s = fp16(absmax / 127),   |x| <= absmax,
 * so the quotient cannot leave [-127.07, 127.07]: saturation is not needed, the residual is always
 * finite, and the integer can be read from the low byte of (q + 1.5 * 2^23), whose single
 * round-to-nearest-even addition is rint(q):
 *
 *     reference:  n = int8(rint(x / s))                          (IEEE fp32 divide, cuda/gemm.cu:16)
 *     fast:       y = 1/s;  q0 = x*y;  r = fma(-s, q0, x);  q1 = fma(r, y, q0);
 *                 n = low byte of the bit pattern of (q1 + 12582912.0f)
 *
 * for EVERY finite fp16 absmax with a normal scale and EVERY fp16 x with |x| <= absmax, and every
 * fp16 NaN x (the absmax ignores NaN elements; the reference build maps NaN to 0, and so does the
 * low byte of a propagated NaN).  Prints the number of mismatching pairs; exits non-zero if any.
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

static float h2f(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16, exp = (h >> 10) & 0x1f, man = h & 0x3ffu, bits;
    if (exp == 0) {
        float v = (float)man * 5.9604644775390625e-08f;
        memcpy(&bits, &v, 4);
        bits |= sign;
    } else if (exp == 31) bits = sign | 0x7f800000u | (man << 13);
    else bits = sign | ((exp + 112) << 23) | (man << 13);
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* fp32 -> fp16, round to nearest even (finite, non-negative inputs below the fp16 range's end) */
static uint16_t f2h(float f) {
    uint32_t b;
    memcpy(&b, &f, 4);
    int32_t e = (int32_t)((b >> 23) & 0xff) - 127 + 15;
    uint32_t m = b & 0x7fffffu;
    if (e >= 31) return 0x7c00;
    if (e <= 0) {
        if (e < -10) return 0;
        m |= 0x800000u;
        const int sh = 14 - e;
        uint32_t r = m >> sh, rem = m & ((1u << sh) - 1), half = 1u << (sh - 1);
        if (rem > half || (rem == half && (r & 1))) ++r;
        return (uint16_t)r;
    }
    uint32_t r = ((uint32_t)e << 10) | (m >> 13), rem = m & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (r & 1))) ++r;
    return (uint16_t)r;
}

static inline int sat_i8(float d) {
    if (d != d) return 0;
    float q = rintf(d);
    if (q < -128.0f) q = -128.0f;
    if (q > 127.0f) q = 127.0f;
    return (int)q;
}

static inline int fast_i8(float x, float s, float y) {
    const float q0 = x * y;
    const float r = fmaf(-s, q0, x);
    const float q1 = fmaf(r, y, q0);
    volatile float t = q1 + 12582912.0f;
    float tt = t;
    uint32_t b;
    memcpy(&b, &tt, 4);
    return (int)(int8_t)(b & 0xffu);
}

int main(void) {
    long long bad = 0, pairs = 0, rows = 0;
#pragma omp parallel for schedule(dynamic, 64) reduction(+ : bad, pairs, rows)
    for (int ai = 0; ai < 0x7c00; ++ai) {                  /* every finite non-negative absmax */
        const float a = h2f((uint16_t)ai);
        const uint16_t sb = f2h(a / 127.0f);
        if (sb < 0x0400 || sb > 0x7bff) continue;          /* the short sequence is used for normal scales only */
        const float s = h2f(sb);
        volatile float one = 1.0f;
        const float y = one / s;
        ++rows;
        for (int xi = 0; xi < 65536; ++xi) {
            const int mag = xi & 0x7fff;
            if (mag > ai && mag <= 0x7c00) continue;       /* |x| > absmax (or inf): cannot be in this row */
            const float x = h2f((uint16_t)xi);
            const int ref = sat_i8(x / s), fast = fast_i8(x, s, y);
            if (ref != fast) {
                if (bad < 5) fprintf(stderr, "mismatch absmax=%04x x=%04x s=%04x ref=%d fast=%d\n", ai, xi, sb, ref, fast);
                ++bad;
            }
            ++pairs;
        }
    }
    printf("%lld rows, %lld pairs, %lld mismatches\n", rows, pairs, bad);
    return bad != 0;
}
