/*
 * CPU restatement of the reference's int8 quantized-GEMM inference path -- TEST INFRASTRUCTURE.
 *
 * This file is the checker, not the product: only tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py may build, load or call it.  Nothing under cpm_kernels_amd/
 * may depend on it.
 *
 * Each function restates, in plain scalar C on host arrays, the arithmetic of one CUDA kernel
 * of OpenBMB/cpm_kernels (cited as file:line of the reference tree).  fp16 values are carried
 * as uint16_t bit patterns and converted in software (no compiler fp16 support is assumed),
 * fp32 arithmetic is IEEE single precision in round-to-nearest-even, the same as the device.
 *
 * How each function is pinned (the checks live in tests/test_oracle.py):
 *   half conversions ........ exhaustive against numpy.float16 (all 65536 patterns; float->half
 *                             on every half-way point and 10^6 random floats)
 *   calc_scale / round ...... closed forms in numpy on random + adversarial rows (ties at .5,
 *                             zero rows, subnormal scales); exhaustive absmax sweep; the
 *                             double-vs-float divide of the reference proven equal exhaustively
 *   gemm_int8 / gemv dot .... brute force vs exact float64 BLAS products (exact: k*128^2 < 2^53),
 *                             all four transpose combinations and both broadcast sides
 *   gemm_scale .............. closed form in numpy float32 (same multiplication order)
 *   gemv_broadcast_mat_int8 . equals gemm_int8 + gemm_scale on the same operands
 *                             (the invariant the reference tests, tests/test_gemv.py:49-59)
 *   layernorm / softmax ..... float64 textbook formulas, torch.softmax, closed-form special
 *                             cases (constant column, one-hot with -inf, all -inf -> 0), m=1
 *   gelu .................... float64 tanh form over all 65536 inputs
 *   position buckets ........ the HF-T5 formula and an exact integer-power formulation for
 *                             every (num_buckets, max_distance, bidirectional) of the
 *                             reference's tests (tests/test_position_embedding.py:6-13)
 *   arith / mask ............ exact float64 closed forms
 * Parity unpinned (undefined behaviour in the reference): float->int8
 * conversion of quotients outside [-128,127] and of NaN (cuda/gemm.cu:16); saturation and
 * NaN->0 are this build's choice.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

/* ---- IEEE binary16 <-> binary32/64 in software ------------------------------------------- */
static float h2f(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1f, man = h & 0x3ffu, bits;
    if (exp == 0) {
        if (man == 0) bits = sign;
        else { /* subnormal: value = man * 2^-24 */
            float v = (float)man * 5.9604644775390625e-08f;
            memcpy(&bits, &v, 4);
            bits |= sign;
        }
    } else if (exp == 31) bits = sign | 0x7f800000u | (man << 13);
    else bits = sign | ((exp + 112) << 23) | (man << 13);
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* round-to-nearest-even double -> half (single rounding; floats pass through exactly) */
static uint16_t d2h(double d) {
    uint64_t b;
    memcpy(&b, &d, 8);
    uint16_t sign = (uint16_t)((b >> 48) & 0x8000u);
    int64_t e = (int64_t)((b >> 52) & 0x7ff);
    uint64_t man = b & 0xfffffffffffffull;
    if (e == 0x7ff) return (uint16_t)(sign | 0x7c00u | (man ? 0x200u : 0));   /* inf / nan */
    if (e == 0) return sign;                       /* double subnormal: far below half range */
    int64_t he = e - 1023 + 15;                    /* biased half exponent */
    man |= 1ull << 52;                             /* explicit leading one: 53-bit significand */
    int shift;                                     /* bits to drop from the 53-bit significand */
    if (he >= 31) return (uint16_t)(sign | 0x7c00u);
    if (he <= 0) {                                 /* half subnormal or underflow */
        shift = 42 + (int)(1 - he);
        he = 0;
        if (shift > 54) return sign;               /* below half of the smallest subnormal */
    } else shift = 42;
    uint64_t q = man >> shift, rem = man & ((1ull << shift) - 1), half = 1ull << (shift - 1);
    if (rem > half || (rem == half && (q & 1))) q++;
    /* q holds the significand with the implicit bit (normal) or without (subnormal); a carry
       out of the mantissa field correctly bumps the exponent, up to infinity */
    uint32_t out = (he > 0) ? (uint32_t)(((uint64_t)(he - 1) << 10) + q) : (uint32_t)q;
    if (out >= 0x7c00u) out = 0x7c00u;
    return (uint16_t)(sign | out);
}
static uint16_t f2h(float f) { return d2h((double)f); }

/* exported for the conversion tests */
void o_half_to_float(int64_t n, const uint16_t* h, float* f) { for (int64_t i = 0; i < n; ++i) f[i] = h2f(h[i]); }
void o_float_to_half(int64_t n, const float* f, uint16_t* h) { for (int64_t i = 0; i < n; ++i) h[i] = f2h(f[i]); }
void o_double_to_half(int64_t n, const double* d, uint16_t* h) { for (int64_t i = 0; i < n; ++i) h[i] = d2h(d[i]); }

/* (int8_t) nearbyintf(x / s): IEEE fp32 divide, round-half-even (cuda/gemm.cu:16).  Out-of-range
 * and NaN conversions are undefined in the reference; saturate / 0 here (see file header). */
static int8_t quant(float x, float s) {
    float d = x / s;
    if (d != d) return 0;
    float r = nearbyintf(d);
    if (r > 127.0f) r = 127.0f;
    if (r < -128.0f) r = -128.0f;
    return (int8_t)r;
}

/* cuda/gemm.cu:60-76 -- out[b,i] = half(max_j |mat[b,i,j]| / 127.0): the reference divides the
 * float maximum by a double literal and passes the double to __float2half (double -> float ->
 * half).  Restated literally. */
static uint16_t scale_of(float mx) { return f2h((float)((double)mx / 127.0)); }

/* The device's fmaxf returns the other operand for ANY NaN operand (cuda/gemm.cu:68-72 relies on
 * it: a NaN element takes no part in the maximum).  The host's fmaxf does so for quiet NaNs only
 * and hands a signalling one on as NaN, so the NaN test is spelled out here. */
static float max_skip_nan(float v, float mx) { return (v != v) ? mx : fmaxf(v, mx); }

void o_gemm_calc_scale(int32_t batch, int32_t n, int32_t m, const uint16_t* mat, uint16_t* out) {
    for (int64_t r = 0; r < (int64_t)batch * n; ++r) {
        float mx = 0.0f;
        for (int32_t j = 0; j < m; ++j) mx = max_skip_nan(fabsf(h2f(mat[r * m + j])), mx);
        out[r] = scale_of(mx);
    }
}

/* cuda/gemm.cu:79-98 -- out[b,j] = half(max_i |in[b,i,j]| / 127.0) */
void o_gemm_calc_scale_transpose(int32_t batch, int32_t n, int32_t m, const uint16_t* mat, uint16_t* out) {
    for (int32_t b = 0; b < batch; ++b)
        for (int32_t j = 0; j < m; ++j) {
            float mx = 0.0f;
            for (int32_t i = 0; i < n; ++i) mx = max_skip_nan(fabsf(h2f(mat[((int64_t)b * n + i) * m + j])), mx);
            out[(int64_t)b * m + j] = scale_of(mx);
        }
}

/* cuda/gemm.cu:6-18 */
void o_gemm_round(int32_t batch, int32_t n, int32_t m, const uint16_t* mat, const uint16_t* scale, int8_t* out) {
    for (int64_t r = 0; r < (int64_t)batch * n; ++r) {
        float s = h2f(scale[r]);
        for (int32_t j = 0; j < m; ++j) out[r * m + j] = quant(h2f(mat[r * m + j]), s);
    }
}

/* cuda/gemm.cu:22-33 */
void o_gemm_round_transpose(int32_t batch, int32_t n, int32_t m, const uint16_t* mat, const uint16_t* scale,
                            int8_t* out) {
    for (int32_t b = 0; b < batch; ++b)
        for (int32_t i = 0; i < n; ++i)
            for (int32_t j = 0; j < m; ++j) {
                int64_t o = ((int64_t)b * n + i) * m + j;
                out[o] = quant(h2f(mat[o]), h2f(scale[(int64_t)b * m + j]));
            }
}

/* cuda/gemm.cu:37-57 -- (float)acc * scale_x * scale_y, left to right */
void o_gemm_scale(int32_t batch, int32_t n, int32_t m, const int32_t* mat, const uint16_t* scale_x,
                  const uint16_t* scale_y, uint16_t* out, int bcx, int bcy) {
    for (int32_t b = 0; b < batch; ++b)
        for (int32_t i = 0; i < n; ++i) {
            float sx = h2f(scale_x[bcx ? i : (int64_t)b * n + i]);
            const uint16_t* sy = bcy ? scale_y : scale_y + (int64_t)b * m;
            for (int32_t j = 0; j < m; ++j) {
                int64_t o = ((int64_t)b * n + i) * m + j;
                float v = (float)mat[o] * sx;
                v = v * h2f(sy[j]);
                out[o] = f2h(v);
            }
        }
}

/* cuda/gemm.cu:176-189 */
void o_gemm_scale_x(int32_t batch, int32_t n, int32_t m, const int32_t* mat, const uint16_t* scale_x, uint16_t* out) {
    for (int64_t r = 0; r < (int64_t)batch * n; ++r) {
        float sx = h2f(scale_x[r]);
        for (int32_t j = 0; j < m; ++j) out[r * m + j] = f2h(sx * (float)mat[r * m + j]);
    }
}

/* cuda/gemm.cu:192-205 */
void o_gemm_scale_y(int32_t batch, int32_t n, int32_t m, const int32_t* mat, const uint16_t* scale_y, uint16_t* out) {
    for (int32_t b = 0; b < batch; ++b)
        for (int32_t i = 0; i < n; ++i)
            for (int32_t j = 0; j < m; ++j) {
                int64_t o = ((int64_t)b * n + i) * m + j;
                out[o] = f2h((float)mat[o] * h2f(scale_y[(int64_t)b * m + j]));
            }
}

/* cpm_kernels/kernels/gemm.py:127-186 -- the cuBLASLt call, restated from its column-major
 * layouts: out[b, j, i] = sum_kk opA[i,kk] * opB[kk,j] with
 *   A memory (k,m) row-major if !aT else (m,k);  B memory (n,k) row-major if !bT else (k,n);
 *   batch stride 0 for an operand whose batch is 1 (:152-155). */
void o_gemm_int8(int32_t m, int32_t k, int32_t n, int32_t batchA, int32_t batchB, int aT, int bT,
                 const int8_t* A, const int8_t* B, int32_t* out) {
    int32_t batch = batchA > batchB ? batchA : batchB;
    for (int32_t b = 0; b < batch; ++b) {
        const int8_t* a = A + (batchA == 1 ? 0 : (int64_t)b * m * k);
        const int8_t* bb = B + (batchB == 1 ? 0 : (int64_t)b * n * k);
        for (int32_t j = 0; j < n; ++j)
            for (int32_t i = 0; i < m; ++i) {
                int32_t acc = 0;
                for (int32_t kk = 0; kk < k; ++kk) {
                    int32_t av = aT ? a[(int64_t)i * k + kk] : a[(int64_t)kk * m + i];
                    int32_t bv = bT ? bb[(int64_t)kk * n + j] : bb[(int64_t)j * k + kk];
                    acc += av * bv;
                }
                out[((int64_t)b * n + j) * m + i] = acc;
            }
    }
}

/* cuda/gemv.cu:26-40 and :43-54 are the row forms above with batch rows of length n */
void o_gemv_calc_scale(int32_t batch, int32_t n, const uint16_t* vec, uint16_t* out) {
    o_gemm_calc_scale(1, batch, n, vec, out);
}
void o_gemv_round(int32_t batch, int32_t n, const uint16_t* vec, const uint16_t* scale, int8_t* out) {
    o_gemm_round(1, batch, n, vec, scale, out);
}

/* cuda/gemv.cu:57-76 */
void o_gemv_broadcast_mat_int8(int32_t batch, int32_t dim_out, int32_t dim_in, const uint16_t* scale_mat,
                               const int8_t* mat, const uint16_t* scale_vec, const int8_t* vec, uint16_t* out) {
    for (int32_t b = 0; b < batch; ++b)
        for (int32_t o = 0; o < dim_out; ++o) {
            int32_t acc = 0;
            for (int32_t kk = 0; kk < dim_in; ++kk)
                acc += (int32_t)mat[(int64_t)o * dim_in + kk] * (int32_t)vec[(int64_t)b * dim_in + kk];
            float v = (float)acc * h2f(scale_vec[b]);
            v = v * h2f(scale_mat[o]);
            out[(int64_t)b * dim_out + o] = f2h(v);
        }
}

/* cuda/layernorm.cu:6-71 -- over dim 1.  Sums are accumulated in double (the reference uses a
 * hierarchical fp32 sum, "to achieve higher precision", :19); everything after the sums is the
 * reference's fp32 sequence. */
void o_layernorm_forward(int32_t batch, int32_t n, int32_t m, const uint16_t* mat, uint16_t* out, float eps,
                         int rd_mean) {
    for (int32_t b = 0; b < batch; ++b)
        for (int32_t j = 0; j < m; ++j) {
            double s = 0.0, s2 = 0.0;
            for (int32_t i = 0; i < n; ++i) {
                double x = (double)h2f(mat[((int64_t)b * n + i) * m + j]);
                s += x;
                s2 += x * x;
            }
            float var = (float)s2 / (float)n, mean = 0.0f;
            if (rd_mean) {
                mean = (float)s / (float)n;
                var -= mean * mean;
            }
            float rstd = 1.0f / sqrtf(var + eps);
            for (int32_t i = 0; i < n; ++i) {
                int64_t o = ((int64_t)b * n + i) * m + j;
                out[o] = f2h((h2f(mat[o]) - mean) * rstd);
            }
        }
}

/* cuda/softmax.cu:6-43 -- over dim 1 */
void o_softmax_forward(int32_t batch, int32_t n, int32_t m, const uint16_t* in, uint16_t* out) {
    for (int32_t b = 0; b < batch; ++b)
        for (int32_t j = 0; j < m; ++j) {
            float mx = -INFINITY;
            for (int32_t i = 0; i < n; ++i) mx = fmaxf(h2f(in[((int64_t)b * n + i) * m + j]), mx);
            mx = fmaxf(mx, -1e6f);
            double sum = 0.0;
            for (int32_t i = 0; i < n; ++i) sum += (double)expf(h2f(in[((int64_t)b * n + i) * m + j]) - mx);
            float fsum = (float)sum + 1e-10f;
            for (int32_t i = 0; i < n; ++i) {
                int64_t o = ((int64_t)b * n + i) * m + j;
                out[o] = f2h(expf(h2f(in[o]) - mx) / fsum);
            }
        }
}

/* cuda/gelu.cu:6-17 -- double literals around a float tanhf */
void o_gelu_forward(int64_t total, const uint16_t* mat, uint16_t* out) {
    for (int64_t i = 0; i < total; ++i) {
        float x = h2f(mat[i]);
        x = 0.5 * x * (1.0 + tanhf(0.7978845608028654 * x * (1.0 + 0.044715 * x * x)));
        out[i] = f2h(x);
    }
}

/* cuda/position_bucket.cu:6-21 */
void o_position_embedding_init(int32_t num_buckets, int32_t max_distance, int32_t* out, int bidirectional) {
    int32_t part_buckets = num_buckets / (bidirectional ? 2 : 1);
    int32_t exact_buckets = part_buckets / 2;
    int32_t log_buckets = part_buckets - exact_buckets;
    float v = logf(max_distance / exact_buckets);
    for (int32_t i = 0; i < max_distance; ++i) {
        if (i < exact_buckets) out[i] = i;
        else out[i] = (int32_t)(logf((float)i / (float)exact_buckets) / v * log_buckets) + exact_buckets;
    }
}

static int32_t bucket_of(int32_t rel, int32_t num_buckets, int32_t max_distance, const int32_t* map, int bidi) {
    int32_t off = 0;
    if (rel < 0) {
        if (bidi) { rel = -rel; off = num_buckets / 2; }
        else rel = 0;
    }
    if (rel >= max_distance) rel = max_distance - 1;
    return map[rel] + off;
}

/* cuda/position_bucket.cu:25-54 */
void o_position_embedding_forward(int32_t query_len, int32_t key_len, int32_t num_buckets, int32_t max_distance,
                                  int32_t num_head, const int32_t* map, const uint16_t* weight, uint16_t* out,
                                  int bidirectional) {
    for (int32_t k = 0; k < key_len; ++k)
        for (int32_t q = 0; q < query_len; ++q) {
            int32_t bucket = bucket_of(q - k, num_buckets, max_distance, map, bidirectional);
            for (int32_t h = 0; h < num_head; ++h)
                out[((int64_t)h * key_len + k) * query_len + q] = weight[(int64_t)h * num_buckets + bucket];
        }
}

/* cuda/position_bucket.cu:105-133 */
void o_position_embedding_step(int32_t query_pos, int32_t key_len, int32_t num_buckets, int32_t max_distance,
                               int32_t num_head, const int32_t* map, const uint16_t* weight, uint16_t* out,
                               int bidirectional) {
    for (int32_t k = 0; k < key_len; ++k) {
        int32_t bucket = bucket_of(query_pos - k, num_buckets, max_distance, map, bidirectional);
        for (int32_t h = 0; h < num_head; ++h) out[(int64_t)h * key_len + k] = weight[(int64_t)h * num_buckets + bucket];
    }
}

/* cuda/arith.cu:97-112 -- __hfma2: one rounding.  The product x*a of two fp16 values has at most
 * 22 significant bits and is exact in double.  Adding b is exact in double as well whenever the
 * product matters to the result (a finite result keeps the product below 2^17 and b's last bit
 * is at least 2^-24: a span of 41 bits); where the product lies further below b than a double
 * holds, the double sum is b or a double next to it, and b, itself an fp16 value, is far from
 * any fp16 rounding boundary.  Either way d2h of the double sum equals the single rounding of
 * the fused operation (tests/test_oracle.py checks it against exact rational arithmetic). */
void o_arith_ln_mul_add(int32_t batch, int32_t n, int32_t m, const uint16_t* x, const uint16_t* alpha,
                        const uint16_t* beta, uint16_t* out) {
    for (int32_t b = 0; b < batch; ++b)
        for (int32_t i = 0; i < n; ++i) {
            double a = (double)h2f(alpha[i]), be = (double)h2f(beta[i]);
            for (int32_t j = 0; j < m; ++j) {
                int64_t o = ((int64_t)b * n + i) * m + j;
                out[o] = d2h((double)h2f(x[o]) * a + be);
            }
        }
}

/* cuda/arith.cu:115-127 -- __hmul2 */
void o_arith_ln_mul(int32_t batch, int32_t n, int32_t m, const uint16_t* x, const uint16_t* alpha, uint16_t* out) {
    for (int32_t b = 0; b < batch; ++b)
        for (int32_t i = 0; i < n; ++i) {
            double a = (double)h2f(alpha[i]);
            for (int32_t j = 0; j < m; ++j) {
                int64_t o = ((int64_t)b * n + i) * m + j;
                out[o] = d2h((double)h2f(x[o]) * a);
            }
        }
}

/* cuda/arith.cu:19-30 -- __hadd2 */
void o_arith_element_add(int64_t total, const uint16_t* x, const uint16_t* y, uint16_t* out) {
    for (int64_t i = 0; i < total; ++i) out[i] = d2h((double)h2f(x[i]) + (double)h2f(y[i]));
}

/* cuda/mask.cu:6-23 */
void o_mask(int32_t batch, int32_t n, int32_t m, const uint16_t* x, const int8_t* mask, float value, uint16_t* out) {
    uint16_t hv = f2h(value);
    for (int32_t b = 0; b < batch; ++b)
        for (int32_t i = 0; i < n; ++i)
            for (int32_t j = 0; j < m; ++j) {
                int64_t o = ((int64_t)b * n + i) * m + j;
                out[o] = mask[(int64_t)b * m + j] == 0 ? hv : x[o];
            }
}
