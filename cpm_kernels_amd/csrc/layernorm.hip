// Normalisation over dim 1 of (batch, n, m) fp16 and over contiguous rows (decode step):
//   mean = rd_mean ? sum x / n : 0;  var = sum x^2 / n - mean^2;
//   y = fp16( (x - mean) * rsqrt(var + eps) )            (cuda/layernorm.cu:6-71, :343-381)
// optionally followed, on the fp16-rounded y, by the affine of cu_arith_ln_mul_add /
// cu_arith_ln_mul (cuda/arith.cu:97-127): fp16 fma(y, alpha[i], beta[i]) or y * alpha[i].
#include "dim1.h"

namespace cpmk {

__device__ inline half8_t affine8(half8_t y, half_t a, half_t b, bool has_beta) {
    half8_t o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = has_beta ? __builtin_fmaf16(y[e], a, b) : (half_t)(y[e] * a);
    return o;
}

// Single pass: the whole (n x LPR*8) column tile lives in registers.
template <int NT, int LPR, int R>
__global__ __launch_bounds__(NT) void k_layernorm_tile(int32_t n, int32_t m, int32_t tiles_per_batch,
                                                       const half_t* mat, half_t* out,
                                                       const half_t* __restrict__ alpha,
                                                       const half_t* __restrict__ beta, float eps,
                                                       int rd_mean) {
    using T = ColTile<NT, LPR, R>;
    __shared__ float lds[(T::NW + 1) * T::COLS * 2];
    const uint32_t t = xcd_remap(blockIdx.x, gridDim.x);
    const uint32_t b = t / tiles_per_batch, ct = t - b * tiles_per_batch;
    const int32_t col0 = ct * T::COLS + (threadIdx.x % LPR) * 8;
    const int64_t boff = (int64_t)b * n * m;

    half8_t v[R];
    coltile_load<NT, LPR, R>(v, mat + boff, n, m, col0, (half_t)0.0f);

    float s[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) s[e] = 0.0f;
#pragma unroll
    for (int p = 0; p < R; ++p)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float x = (float)v[p][e];
            s[e] += x;
            s[8 + e] += x * x;
        }
    coltile_reduce<NT, LPR, 2, false>(s, lds);

    float mean[8], rstd[8];
    const float fn = (float)n;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        float var = s[8 + e] / fn;
        mean[e] = 0.0f;
        if (rd_mean) {
            mean[e] = s[e] / fn;
            var -= mean[e] * mean[e];
        }
        rstd[e] = rsqrtf(var + eps);
    }
    const int rg = threadIdx.x / LPR;
#pragma unroll
    for (int p = 0; p < R; ++p) {
        half8_t y;
#pragma unroll
        for (int e = 0; e < 8; ++e) y[e] = round_f16(((float)v[p][e] - mean[e]) * rstd[e]);
        if (alpha != nullptr) {
            const int32_t row = p * T::RPP + rg;
            if (row < n) y = affine8(y, alpha[row], beta ? beta[row] : (half_t)0.0f, beta != nullptr);
        }
        v[p] = y;
    }
    coltile_store<NT, LPR, R>(v, out + boff, n, m, col0);
}

// Tall columns (n up to 16 * 1024 with 128-byte row segments).  A register tile can hold
// 1024 rows of 64 columns; narrower tiles would hold more rows but touch only part of every
// cache line, and the partial lines cost more L2 bandwidth than HBM has.  So the n rows of a
// 64-column tile are split over PARTS = ceil(n / 1024) workgroups that run side by side on one
// XCD: each keeps its own 1024 rows in registers and streams the other parts' rows once, only
// to accumulate the column statistics (those reads are L2 hits: a sibling fetched or is
// fetching the same lines).  No workgroup waits for another, so there is nothing to deadlock.
template <int NT, int R>
__global__ __launch_bounds__(NT) void k_layernorm_tall(int32_t n, int32_t m, int32_t tiles_per_batch, int32_t parts,
                                                       const half_t* mat, half_t* out,
                                                       const half_t* __restrict__ alpha,
                                                       const half_t* __restrict__ beta, float eps, int rd_mean) {
    constexpr int LPR = 8;
    using T = ColTile<NT, LPR, R>;
    __shared__ float lds[(T::NW + 1) * T::COLS * 2];
    const uint32_t t = xcd_remap(blockIdx.x, gridDim.x);
    const uint32_t part = t % parts, tile = t / parts;
    const uint32_t b = tile / tiles_per_batch, ct = tile - b * tiles_per_batch;
    const int32_t col0 = ct * T::COLS + (threadIdx.x % LPR) * 8;
    const int64_t boff = (int64_t)b * n * m;
    const int32_t own0 = part * T::ROWS;                 // first row this workgroup normalises
    const int32_t own_n = min(T::ROWS, n - own0);        // > 0 by construction

    half8_t v[R];
    coltile_load<NT, LPR, R>(v, mat + boff + (int64_t)own0 * m, own_n, m, col0, (half_t)0.0f);
    float s[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) s[e] = 0.0f;
    // the other parts' rows: statistics only
    const int rg = threadIdx.x / LPR;
    if (col0 < m) {
        for (int32_t r0 = 0; r0 < n; r0 += T::RPP * 4) {
            half8_t w[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int32_t row = r0 + u * T::RPP + rg;
                const bool mine = row >= own0 && row < own0 + T::ROWS;
#pragma unroll
                for (int e = 0; e < 8; ++e) w[u][e] = (half_t)0.0f;
                if (row < n && !mine) w[u] = *reinterpret_cast<const half8_t*>(mat + boff + ((uint32_t)row * (uint32_t)m + (uint32_t)col0));
            }
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float x = (float)w[u][e];
                    s[e] += x;
                    s[8 + e] += x * x;
                }
        }
    }
#pragma unroll
    for (int p = 0; p < R; ++p)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float x = (float)v[p][e];
            s[e] += x;
            s[8 + e] += x * x;
        }
    coltile_reduce<NT, LPR, 2, false>(s, lds);

    float mean[8], rstd[8];
    const float fn = (float)n;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        float var = s[8 + e] / fn;
        mean[e] = 0.0f;
        if (rd_mean) {
            mean[e] = s[e] / fn;
            var -= mean[e] * mean[e];
        }
        rstd[e] = rsqrtf(var + eps);
    }
#pragma unroll
    for (int p = 0; p < R; ++p) {
        half8_t y;
#pragma unroll
        for (int e = 0; e < 8; ++e) y[e] = round_f16(((float)v[p][e] - mean[e]) * rstd[e]);
        if (alpha != nullptr) {
            const int32_t row = own0 + p * T::RPP + rg;
            if (row < n) y = affine8(y, alpha[row], beta ? beta[row] : (half_t)0.0f, beta != nullptr);
        }
        v[p] = y;
    }
    coltile_store<NT, LPR, R>(v, out + boff + (int64_t)own0 * m, own_n, m, col0);
}

// Generic fallback (any n, m, alignment): 64 columns x 4 row groups per workgroup, two
// passes over global memory; the statistics are complete before the first store, and each
// element is re-read by the thread that overwrites it, so out may alias mat.
__global__ __launch_bounds__(256) void k_layernorm_generic(int32_t n, int32_t m, const half_t* mat, half_t* out,
                                                           const half_t* __restrict__ alpha,
                                                           const half_t* __restrict__ beta, float eps,
                                                           int rd_mean) {
    __shared__ float red[2][4][64];
    const int c = threadIdx.x & 63, rg = threadIdx.x >> 6;
    const int32_t col = blockIdx.x * 64 + c;
    const int64_t boff = (int64_t)blockIdx.y * n * m;
    float s = 0.0f, s2 = 0.0f;
    if (col < m) {
        for (int32_t i = rg; i < n; i += 4) {
            const float x = (float)mat[boff + (int64_t)i * m + col];
            s += x;
            s2 += x * x;
        }
    }
    red[0][rg][c] = s;
    red[1][rg][c] = s2;
    __syncthreads();
    s = red[0][0][c] + red[0][1][c] + red[0][2][c] + red[0][3][c];
    s2 = red[1][0][c] + red[1][1][c] + red[1][2][c] + red[1][3][c];
    const float fn = (float)n;
    float var = s2 / fn, mean = 0.0f;
    if (rd_mean) {
        mean = s / fn;
        var -= mean * mean;
    }
    const float rstd = rsqrtf(var + eps);
    if (col < m) {
        for (int32_t i = rg; i < n; i += 4) {
            const int64_t o = boff + (int64_t)i * m + col;
            half_t y = round_f16(((float)mat[o] - mean) * rstd);
            if (alpha != nullptr) y = beta ? __builtin_fmaf16(y, alpha[i], beta[i]) : (half_t)(y * alpha[i]);
            out[o] = y;
        }
    }
}

// Contiguous rows (batch, n): one 256-thread workgroup per row.
__global__ __launch_bounds__(256) void k_layernorm_rows(int32_t n, const half_t* mat, half_t* out, float eps,
                                                        int rd_mean) {
    __shared__ float red[4];
    const half_t* p = mat + (int64_t)blockIdx.x * n;
    half_t* o = out + (int64_t)blockIdx.x * n;
    float s = 0.0f, s2 = 0.0f;
    for (int32_t i = threadIdx.x; i < n; i += 256) {
        const float x = (float)p[i];
        s += x;
        s2 += x * x;
    }
    s = block_sum<4>(s, red);
    s2 = block_sum<4>(s2, red);
    const float fn = (float)n;
    float var = s2 / fn, mean = 0.0f;
    if (rd_mean) {
        mean = s / fn;
        var -= mean * mean;
    }
    const float rstd = rsqrtf(var + eps);
    for (int32_t i = threadIdx.x; i < n; i += 256) o[i] = round_f16(((float)p[i] - mean) * rstd);
}

template <int LPR, int R>
static void launch_tile(int32_t batch, int32_t n, int32_t m, const half_t* mat, half_t* out, const half_t* alpha,
                        const half_t* beta, float eps, int rd_mean, hipStream_t st) {
    constexpr int NT = 1024;
    const int32_t tiles = (int32_t)ceil_div(m, LPR * 8);
    hipLaunchKernelGGL((k_layernorm_tile<NT, LPR, R>), dim3((unsigned)((int64_t)tiles * batch)), dim3(NT), 0, st, n,
                       m, tiles, mat, out, alpha, beta, eps, rd_mean);
}

template <int LPR>
static bool launch_tile_r(int r, int32_t batch, int32_t n, int32_t m, const half_t* mat, half_t* out,
                          const half_t* alpha, const half_t* beta, float eps, int rd_mean, hipStream_t st) {
    if (r <= 1) launch_tile<LPR, 1>(batch, n, m, mat, out, alpha, beta, eps, rd_mean, st);
    else if (r <= 2) launch_tile<LPR, 2>(batch, n, m, mat, out, alpha, beta, eps, rd_mean, st);
    else if (r <= 4) launch_tile<LPR, 4>(batch, n, m, mat, out, alpha, beta, eps, rd_mean, st);
    else if (r <= 8) launch_tile<LPR, 8>(batch, n, m, mat, out, alpha, beta, eps, rd_mean, st);
    else return false;
    return true;
}

static int layernorm_dispatch(int32_t batch, int32_t n, int32_t m, const void* mat, void* out, const void* alpha,
                              const void* beta, float eps, int rd_mean, hipStream_t st) {
    if (batch < 0 || n < 0 || m < 0) return CPMK_EBADARG;
    if ((int64_t)batch * n * m == 0) return 0;
    const half_t* x = (const half_t*)mat;
    half_t* y = (half_t*)out;
    const half_t* al = (const half_t*)alpha;
    const half_t* be = (const half_t*)beta;
    if (m == 1 && alpha == nullptr) {
        hipLaunchKernelGGL(k_layernorm_rows, dim3((unsigned)batch), dim3(256), 0, st, n, x, y, eps, rd_mean);
        return launch_status();
    }
    if (m % 8 == 0 && aligned16(mat) && aligned16(out) && (int64_t)n * m < (1ll << 31)) {
        // widest row segment whose tile still fits the register budget (at most 8 pieces per lane)
        bool ok = false;
        if (n > 128 * 8 && n <= 16 * 1024 && m >= 64 && (const void*)x != (const void*)y) {
            // tall columns: 64-column tiles, n split over side-by-side workgroups.  Not for in-place
            // calls: a workgroup would overwrite rows that a sibling still reads for its statistics.
            const int32_t parts = (int32_t)ceil_div(n, 1024), tiles = (int32_t)ceil_div(m, 64);
            hipLaunchKernelGGL((k_layernorm_tall<1024, 8>), dim3((unsigned)((int64_t)tiles * batch * parts)), dim3(1024), 0,
                               st, n, m, tiles, parts, x, y, al, be, eps, rd_mean);
            return launch_status();
        }
        if (n <= 128 * 8 && m >= 64) ok = launch_tile_r<8>((int)ceil_div(n, 128), batch, n, m, x, y, al, be, eps, rd_mean, st);
        else if (n <= 256 * 8 && m >= 32) ok = launch_tile_r<4>((int)ceil_div(n, 256), batch, n, m, x, y, al, be, eps, rd_mean, st);
        else ok = launch_tile_r<2>((int)ceil_div(n, 512), batch, n, m, x, y, al, be, eps, rd_mean, st);
        if (ok) return launch_status();
    }
    dim3 grid((unsigned)ceil_div(m, 64), (unsigned)batch);
    if (batch > 65535) return CPMK_ETOOBIG;
    hipLaunchKernelGGL(k_layernorm_generic, grid, dim3(256), 0, st, n, m, x, y, al, be, eps, rd_mean);
    return launch_status();
}

}  // namespace cpmk

using namespace cpmk;

extern "C" {

int cpmk_layernorm_forward(int32_t batch, int32_t n, int32_t m, const void* mat, void* out, float eps,
                           int rd_mean, void* stream) {
    clear_stale_error();
    return layernorm_dispatch(batch, n, m, mat, out, nullptr, nullptr, eps, rd_mean, (hipStream_t)stream);
}

int cpmk_layernorm_affine_forward(int32_t batch, int32_t n, int32_t m, const void* mat, const void* alpha,
                                  const void* beta, void* out, float eps, int rd_mean, void* stream) {
    clear_stale_error();
    if (alpha == nullptr) return CPMK_EBADARG;
    return layernorm_dispatch(batch, n, m, mat, out, alpha, beta, eps, rd_mean, (hipStream_t)stream);
}

int cpmk_layernorm_step(int32_t batch, int32_t n, const void* mat, void* out, float eps, int rd_mean,
                        void* stream) {
    clear_stale_error();
    if (batch < 0 || n < 0) return CPMK_EBADARG;
    if ((int64_t)batch * n == 0) return 0;
    hipLaunchKernelGGL(k_layernorm_rows, dim3((unsigned)batch), dim3(256), 0, (hipStream_t)stream, n,
                       (const half_t*)mat, (half_t*)out, eps, rd_mean);
    return launch_status();
}

}  // extern "C"
