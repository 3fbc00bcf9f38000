// Streaming fp16 kernels: GELU, per-channel affine, residual add, padding mask.
// One 16-byte load/store per lane wherever the shape allows it.
#include "common.h"

namespace cpmk {

// Eight halves of a flat tensor: on 16-byte boundaries with the non-temporal hint (WIDE 1), at any address without it
// (WIDE 2: global accesses need no alignment).
__device__ __forceinline__ half8_t flat_load8(const half_t* p, int wide) {
    return wide == 1 ? __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(p)) : load_half8_any(p);
}
__device__ __forceinline__ void flat_store8(half_t* p, half8_t v, int wide) {
    if (wide == 1) __builtin_nontemporal_store(v, reinterpret_cast<half8_t*>(p));
    else store_half8_any(p, v);
}

// cuda/gelu.cu:14 evaluates 0.5 * x * (1 + tanh(c * x * (1 + 0.044715 x^2))), c = sqrt(2/pi), partly in
// double.  With u = c x (1 + 0.044715 x^2) the same function is x / (1 + exp(-2u)), which needs
// one exp2 and one reciprocal in fp32 and, unlike 1 + tanh(u), does not cancel for negative x.
// The fp32 result is within a few ulps of the exact value, so its fp16 rounding is the exact
// one or its neighbour (the bar of the contract is 1e-3 relative).
__device__ inline half_t gelu1(half_t h) {
    const float x = (float)h;
    constexpr float k1 = -2.3022081981462618f;     // -2 log2(e) c
    constexpr float k2 = -0.10294323958011010f;    // -2 log2(e) c * 0.044715
    const float e = __builtin_amdgcn_exp2f(x * __builtin_fmaf(k2, x * x, k1));      // exp(-2u)
    return (half_t)(x * __builtin_amdgcn_rcpf(1.0f + e));
}

__global__ __launch_bounds__(256) void k_gelu(int64_t total, const half_t* mat, half_t* out, int vec) {
    const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (vec) {
        const int64_t e0 = gid * 8;
        if (e0 + 8 <= total) {
            half8_t v = flat_load8(mat + e0, vec);
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = gelu1(v[e]);
            flat_store8(out + e0, v, vec);
        } else {
            for (int64_t i = e0; i < total; ++i) out[i] = gelu1(mat[i]);
        }
    } else if (gid < total) {
        out[gid] = gelu1(mat[gid]);
    }
}

// out[b,i,:] = fma(x, alpha[i], beta[i]) (HAS_BETA) or x * alpha[i], fp16 arithmetic
// (cuda/arith.cu:97-127).  rows = batch*n, channel = row % n.
template <bool HAS_BETA>
__global__ __launch_bounds__(256) void k_ln_affine(int64_t total, int32_t n, int32_t m, const half_t* x,
                                                   const half_t* __restrict__ alpha,
                                                   const half_t* __restrict__ beta, half_t* out, int vec) {
    const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t e0 = vec ? gid * 8 : gid * 2;       // m % 2 == 0 (vec 1: m % 8 == 0)
    if (e0 >= total) return;
    const int32_t ch = (int32_t)((e0 / m) % n);
    const half_t a = alpha[ch];
    const half_t b = HAS_BETA ? beta[ch] : (half_t)0.0f;
    if (vec == 2) {
        // rows that are not whole 16-byte pieces (m >= 8), or buffers off 16-byte boundaries: the tensor is still one
        // contiguous run, so its elements go eight at a time at whatever address they start; the eight may run over
        // the end of a row into the next channel
        if (e0 + 8 <= total) {
            const int32_t left = m - (int32_t)(e0 % m);       // elements of this row from e0 on
            const int32_t ch1 = ch + 1 == n ? 0 : ch + 1;
            const half_t a1 = alpha[ch1];
            const half_t b1 = HAS_BETA ? beta[ch1] : (half_t)0.0f;
            half8_t v = load_half8_any(x + e0);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const half_t ae = e < left ? a : a1, be = e < left ? b : b1;
                v[e] = HAS_BETA ? __builtin_fmaf16(v[e], ae, be) : (half_t)(v[e] * ae);
            }
            store_half8_any(out + e0, v);
        } else {
            for (int64_t i = e0; i < total; ++i) {
                const int32_t c = (int32_t)((i / m) % n);
                out[i] = HAS_BETA ? __builtin_fmaf16(x[i], alpha[c], beta[c]) : (half_t)(x[i] * alpha[c]);
            }
        }
    } else if (vec) {
        half8_t v = __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(x + e0));
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = HAS_BETA ? __builtin_fmaf16(v[e], a, b) : (half_t)(v[e] * a);
        __builtin_nontemporal_store(v, reinterpret_cast<half8_t*>(out + e0));
    } else {
        half2_t v = *reinterpret_cast<const half2_t*>(x + e0);
#pragma unroll
        for (int e = 0; e < 2; ++e) v[e] = HAS_BETA ? __builtin_fmaf16(v[e], a, b) : (half_t)(v[e] * a);
        *reinterpret_cast<half2_t*>(out + e0) = v;
    }
}

__global__ __launch_bounds__(256) void k_add(int64_t total, const half_t* x, const half_t* y, half_t* out, int vec) {
    const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (vec) {
        const int64_t e0 = gid * 8;
        if (e0 + 8 <= total) {
            half8_t a = flat_load8(x + e0, vec);
            half8_t b = flat_load8(y + e0, vec);
            flat_store8(out + e0, a + b, vec);
        } else {
            for (int64_t i = e0; i < total; ++i) out[i] = x[i] + y[i];
        }
    } else if (gid < total) {
        out[gid] = x[gid] + y[gid];
    }
}

// out[b,i,j] = mask[b,j] == 0 ? value : x[b,i,j]      (cuda/mask.cu:6-23)
__global__ __launch_bounds__(256) void k_mask(int64_t total, int32_t n, int32_t m, const half_t* x,
                                              const int8_t* __restrict__ mask, half_t value, half_t* out, int vec) {
    const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t e0 = vec ? gid * 8 : gid;
    if (e0 >= total) return;
    const int64_t row = e0 / m;
    const int32_t j = (int32_t)(e0 - row * m);
    const int8_t* mp = mask + (row / n) * m + j;
    if (vec == 2) {
        // rows that are not whole 16-byte pieces (m >= 8): the tensor is still one contiguous run, so its elements go
        // eight at a time; the eight may run over the end of a row, and each looks up its own mask byte
        if (e0 + 8 <= total) {
            const int wide = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0 ? 1 : 2;
            half8_t v = flat_load8(x + e0, wide);
            const int8_t* m0 = mask + (row / n) * m + j;                   // this row's mask bytes from column j on
            if (j + 8 <= m) {       // the eight share a row: their mask bytes in one load (global loads need no alignment)
                const Byte8Any mk = *reinterpret_cast<const Byte8Any*>(m0);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const uint32_t byte = ((e < 4 ? mk.x : mk.y) >> ((e & 3) * 8)) & 0xffu;
                    if (byte == 0) v[e] = value;
                }
            } else {
                const int8_t* m1 = mask + ((row + 1) / n) * m + (j - m);       // the next row's, addressed by the same index
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if ((j + e < m ? m0 : m1)[e] == 0) v[e] = value;
            }
            flat_store8(out + e0, v, wide);
        } else {
            for (int64_t i = e0; i < total; ++i) {
                const int64_t r2 = i / m;
                out[i] = (mask[(r2 / n) * m + (i - r2 * m)] == 0) ? value : x[i];
            }
        }
    } else if (vec) {
        half8_t v = __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(x + e0));
        const uint2_t mk = *reinterpret_cast<const uint2_t*>(mp);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const uint32_t byte = ((e < 4 ? mk.x : mk.y) >> ((e & 3) * 8)) & 0xffu;
            if (byte == 0) v[e] = value;
        }
        __builtin_nontemporal_store(v, reinterpret_cast<half8_t*>(out + e0));
    } else {
        out[e0] = (mp[0] == 0) ? value : x[e0];
    }
}

}  // namespace cpmk

using namespace cpmk;

extern "C" {

int cpmk_gelu_forward(int32_t batch, int32_t n, const void* mat, void* out, void* stream) {
    clear_stale_error();
    if (batch < 0 || n < 0) return CPMK_EBADARG;
    const int64_t total = (int64_t)batch * n;
    if (total == 0) return 0;
    if (any_null(mat, out)) return CPMK_EBADARG;
    const int vec = aligned16(mat) && aligned16(out) ? 1 : 2;       // (2: buffers off 16-byte boundaries)
    const int64_t g = ceil_div(ceil_div(total, 8), 256);
    hipLaunchKernelGGL(k_gelu, dim3((unsigned)g), dim3(256), 0, (hipStream_t)stream, total, (const half_t*)mat,
                       (half_t*)out, vec);
    return launch_status();
}

static int ln_affine(int32_t batch, int32_t n, int32_t m, const void* inp, const void* alpha, const void* beta,
                     void* out, hipStream_t st) {
    if (batch < 0 || n < 0 || m < 0) return CPMK_EBADARG;
    if (m % 2) return CPMK_EALIGN;   // kernels/arith.py:146,200
    const int64_t total = (int64_t)batch * n * m;
    if (total == 0) return 0;
    if (any_null(inp, alpha, out)) return CPMK_EBADARG;
    const int vec = (m % 8 == 0) && aligned16(inp) && aligned16(out) ? 1 : m >= 8 ? 2 : 0;
    const int64_t g = ceil_div(vec ? ceil_div(total, 8) : total / 2, 256);
    if (beta)
        hipLaunchKernelGGL((k_ln_affine<true>), dim3((unsigned)g), dim3(256), 0, st, total, n, m, (const half_t*)inp,
                           (const half_t*)alpha, (const half_t*)beta, (half_t*)out, vec);
    else
        hipLaunchKernelGGL((k_ln_affine<false>), dim3((unsigned)g), dim3(256), 0, st, total, n, m, (const half_t*)inp,
                           (const half_t*)alpha, (const half_t*)nullptr, (half_t*)out, vec);
    return launch_status();
}

int cpmk_arith_ln_mul_add(int32_t batch, int32_t n, int32_t m, const void* inp, const void* alpha,
                          const void* beta, void* out, void* stream) {
    clear_stale_error();
    if (beta == nullptr) return CPMK_EBADARG;
    return ln_affine(batch, n, m, inp, alpha, beta, out, (hipStream_t)stream);
}

int cpmk_arith_ln_mul(int32_t batch, int32_t n, int32_t m, const void* inp, const void* alpha, void* out,
                      void* stream) {
    clear_stale_error();
    return ln_affine(batch, n, m, inp, alpha, nullptr, out, (hipStream_t)stream);
}

int cpmk_arith_element_add(int32_t batch, int32_t n, const void* x, const void* y, void* out, void* stream) {
    clear_stale_error();
    if (batch < 0 || n < 0) return CPMK_EBADARG;
    if (n % 2) return CPMK_EALIGN;   // kernels/arith.py:53
    const int64_t total = (int64_t)batch * n;
    if (total == 0) return 0;
    if (any_null(x, y, out)) return CPMK_EBADARG;
    const int vec = aligned16(x) && aligned16(y) && aligned16(out) ? 1 : 2;       // (2: buffers off 16-byte boundaries)
    const int64_t g = ceil_div(ceil_div(total, 8), 256);
    hipLaunchKernelGGL(k_add, dim3((unsigned)g), dim3(256), 0, (hipStream_t)stream, total, (const half_t*)x,
                       (const half_t*)y, (half_t*)out, vec);
    return launch_status();
}

int cpmk_mask(int32_t batch, int32_t n, int32_t m, const void* inp, const void* mask, float value, void* out,
              void* stream) {
    clear_stale_error();
    if (batch < 0 || n < 0 || m < 0) return CPMK_EBADARG;
    const int64_t total = (int64_t)batch * n * m;
    if (total == 0) return 0;
    if (any_null(inp, mask, out)) return CPMK_EBADARG;
    int vec = (m % 8 == 0) && aligned16(inp) && aligned16(out) && ((reinterpret_cast<uintptr_t>(mask) & 7u) == 0);
    if (!vec && m >= 8) vec = 2;
    const int64_t g = ceil_div(vec ? ceil_div(total, 8) : total, 256);
    hipLaunchKernelGGL(k_mask, dim3((unsigned)g), dim3(256), 0, (hipStream_t)stream, total, n, m, (const half_t*)inp,
                       (const int8_t*)mask, (half_t)value, (half_t*)out, vec);
    return launch_status();
}

}  // extern "C"
