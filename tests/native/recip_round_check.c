/*
 * Exhaustive proof, on the CPU, that rounding to int8 through a reciprocal and one residual
 * correction equals the reference's divide-then-round (cuda/gemm.cu:16) for EVERY pair of fp16
 * value and fp16 scale:
 *
 *     reference:  q = rint(x / s)                               (IEEE fp32 divide)
 *     fast:       y = 1/s (IEEE, once per row);  q0 = x*y;  r = fma(-s, q0, x);
 *                 q1 = fma(r, y, q0);  q = rint(r finite ? q1 : q0)
 *
 * followed in both cases by saturation to [-128,127] and NaN -> 0.  The device code in
 * csrc/common.h uses exactly these fp32 operations (mul, fma, rint are IEEE on the GPU).
 * Usage: recip_round_check [first_scale_pattern last_scale_pattern]; prints the number of
 * mismatching pairs and exits non-zero if there is one.
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
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

static inline int sat_i8(float d) {
    if (d != d) return 0;
    float q = rintf(d);
    if (q < -128.0f) q = -128.0f;
    if (q > 127.0f) q = 127.0f;
    return (int)q;
}

int main(int argc, char** argv) {
    int s_lo = 0, s_hi = 65535;
    if (argc == 3) { s_lo = atoi(argv[1]); s_hi = atoi(argv[2]); }
    static float xs[65536];
    for (int i = 0; i < 65536; ++i) xs[i] = h2f((uint16_t)i);
    long long bad = 0, pairs = 0;
#pragma omp parallel for schedule(dynamic, 64) reduction(+ : bad, pairs)
    for (int si = s_lo; si <= s_hi; ++si) {
        const float s = xs[si];
        volatile float one = 1.0f;
        const float y = one / s;
        for (int xi = 0; xi < 65536; ++xi) {
            const float x = xs[xi];
            const int ref = sat_i8(x / s);
            const float q0 = x * y;
            const float r = fmaf(-s, q0, x);
            const float q1 = fmaf(r, y, q0);
            const int fast = sat_i8((r - r == 0.0f) ? q1 : q0);
            if (ref != fast) {
                if (bad < 5) fprintf(stderr, "mismatch x=%04x s=%04x ref=%d fast=%d\n", xi, si, ref, fast);
                ++bad;
            }
            ++pairs;
        }
    }
    printf("%lld pairs, %lld mismatches\n", pairs, bad);
    return bad != 0;
}
