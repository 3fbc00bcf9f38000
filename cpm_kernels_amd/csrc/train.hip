// Training-side and remaining elementwise kernels of the reference, forward results and
// gradients (cuda/arith.cu, cuda/gelu.cu:18-45, cuda/gemm.cu:100-172, cuda/layernorm.cu:142-339,
// cuda/softmax.cu:86-114, cuda/position_bucket.cu:56-103, cuda/embedding.cu:38-88).  None of
// them is on the inference hot path; they use 16-byte accesses and fp32 accumulation, and the
// reductions over dim 1 share the register-resident column tile and the team exchange of the
// forward layernorm.
#include "dim1.h"
#include "exchange.h"

namespace cpmk {

// ---------------------------------------------------------------------------------------
// fp16 elementwise family.  BC selects what the second/third operand is indexed by:
//   0 same element, 1 column (idx % n) -- the "batch_*" ops, 2 channel ((idx / m) % n) -- "ln_*".
// The arithmetic is the reference's: one fp16 rounding per __hadd2/__hmul2/__hfma2.
// ---------------------------------------------------------------------------------------
enum : int { kAdd = 0, kMul = 1, kFma = 2, kDiv = 3, kSubDiv = 4 };

__device__ inline half_t ew_apply(int op, half_t x, half_t a, half_t b) {
    switch (op) {
        case kAdd: return (half_t)(x + a);
        case kMul: return (half_t)(x * a);
        case kFma: return __builtin_fmaf16(x, a, b);
        case kDiv: return (half_t)(x * (half_t)(1.0f / (float)a));     // __hmul2(x, __hdiv(1, alpha)); fp32 quotient -> fp16 rounds once
        default: {                                                                   // cu_arith_ln_sub_div
            const float ra = (float)(1.0 / (double)(float)a);
            const float nb = -(float)b * ra;
            return __builtin_fmaf16(x, (half_t)ra, round_f16(nb));
        }
    }
}

// The tensor is seen as rows x cols: BC 0: one row; BC 1: rows = batch, cols = n, a/b indexed by the
// column; BC 2: rows = batch*n, cols = m, a/b indexed by row % n.  blockIdx.x = row * chunks + chunk;
// a thread handles 8 adjacent elements of a row.  ANY false: cols % 8 == 0 and everything 16-byte aligned; true: any
// row length and alignment -- eight elements inside the row still move as one 16-byte access at whatever address they
// start, the piece across the row's end in narrower ones.
template <int OP, int BC, bool ANY>
__global__ __launch_bounds__(256) void k_ew(int64_t cols, uint32_t chunks, int64_t n, const half_t* x, const half_t* __restrict__ a,
                                            const half_t* __restrict__ b, half_t* out) {
    constexpr int V = 8;
    // BC 1: the rows of one chunk of columns run side by side, so a/b are fetched from HBM once
    const uint32_t rows = gridDim.x / chunks;
    const uint32_t chunk = BC == 1 ? blockIdx.x / rows : blockIdx.x % chunks;
    const int64_t row = BC == 1 ? blockIdx.x % rows : blockIdx.x / chunks;
    const int64_t c = ((int64_t)chunk * 256 + threadIdx.x) * V;
    if (c >= cols) return;
    const int64_t i = row * cols + c;
    const int t = !ANY || cols - c >= V ? V : (int)(cols - c);        // elements of this piece inside the row
    const half8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
    auto get = [&](const half_t* p) __attribute__((always_inline)) {
        if constexpr (!ANY) return *reinterpret_cast<const half8_t*>(p);
        else return t == V ? load_half8_any(p) : load_half8_head_any(p, t, zero);
    };
    const half8_t v = get(x + i);
    half8_t av = zero, bv = zero;
    if (BC == 2) {
        const int64_t k = row % n;
        const half_t a1 = a[k], b1 = b ? b[k] : (half_t)0.0f;
#pragma unroll
        for (int e = 0; e < V; ++e) { av[e] = a1; bv[e] = b1; }
    } else {
        const int64_t k = BC == 0 ? i : c;
        av = get(a + k);
        if (b) bv = get(b + k);
    }
    half8_t r;
#pragma unroll
    for (int e = 0; e < V; ++e) r[e] = ew_apply(OP, v[e], av[e], bv[e]);
    if constexpr (!ANY) *reinterpret_cast<half8_t*>(out + i) = r;
    else if (t == V) store_half8_any(out + i, r);
    else store_half8_head_any(out + i, t, r);
}

template <int V>
__global__ __launch_bounds__(256) void k_global_scale(int64_t n, const half_t* inp, float scale, half_t* out) {
    typedef half_t vec_t __attribute__((ext_vector_type(V)));
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * V;
    if (i >= n) return;
    if (V > 1) {
        const vec_t v = *reinterpret_cast<const vec_t*>(inp + i);
        vec_t r;
#pragma unroll
        for (int e = 0; e < V; ++e) r[e] = round_f16((float)v[e] * scale);
        *reinterpret_cast<vec_t*>(out + i) = r;
    } else {
        out[i] = round_f16((float)inp[i] * scale);
    }
}

// cu_gelu_backward: grad = gelu'(x) * grad_out with the reference's constants and cut-off at |x| >= 5
// (cuda/gelu.cu:18-45): gelu'(x) = 0.5 + 0.5 tanh(u) + (0.398942 x + 0.0535161 x^3) sech^2(u),
// u = 0.797885 x + 0.0356774 x^3.  Both hyperbolic terms come from one exponential e = exp(-2|u|):
// sech^2 = 4 e / (1 + e)^2 and 0.5 + 0.5 tanh(u) = 1 / (1 + e) for u >= 0, e / (1 + e) otherwise,
// which has no cancellation where the derivative is small.
__device__ inline half_t gelu_grad1(half_t gh, half_t xh) {
    const float v = (float)gh, x = (float)xh;
    float g;
    if (-5.0f < x && x < 5.0f) {
        const float x3 = x * x * x;
        const float u = 0.797885f * x + 0.0356774f * x3;
        const float e = __builtin_amdgcn_exp2f(-2.8853900817779268f * fabsf(u));       // exp(-2|u|)
        const float r = 1.0f / (1.0f + e);
        const float hp = u < 0.0f ? e * r : r;
        g = hp + (0.398942f * x + 0.0535161f * x3) * (4.0f * e * r * r);
    } else {
        g = x < 0.0f ? 0.0f : 1.0f;
    }
    return round_f16(g * v);
}

template <int V>
__global__ __launch_bounds__(256) void k_gelu_backward(int64_t total, const half_t* grad_out, const half_t* mat, half_t* grad) {
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * V;
    if (i >= total) return;
    if constexpr (V == 8) {
        const half8_t gv = *reinterpret_cast<const half8_t*>(grad_out + i), xv = *reinterpret_cast<const half8_t*>(mat + i);
        half8_t o;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = gelu_grad1(gv[e], xv[e]);
        *reinterpret_cast<half8_t*>(grad + i) = o;
    } else {
        grad[i] = gelu_grad1(grad_out[i], mat[i]);
    }
}

// ---------------------------------------------------------------------------------------
// Sums over everything but one index (fp32 accumulation, one workgroup per output).
// ---------------------------------------------------------------------------------------
// grad[j] = sum_b grad_out[b, j]                                            cu_arith_batch_add_backward
// A lane owns eight adjacent columns: one 16-byte load per row at whatever address the piece starts (global loads need
// no alignment), eight rows requested at a time, the sums in fp32; the piece across the end of the row in narrower
// accesses.  With few columns the rows are dealt to `rgs` (a power of two up to 64) groups of 256 / rgs lanes, whose
// sums are added in group order.
__global__ __launch_bounds__(256) void k_batch_add_backward(int64_t batch, int64_t n, int rgs, const half_t* __restrict__ grad_out,
                                                            half_t* __restrict__ grad) {
    __shared__ float red[2048];                 // [row group][column of the workgroup]
    const int cgs = 256 / rgs, cg = threadIdx.x % cgs, rg = threadIdx.x / cgs;
    const int64_t col = ((int64_t)blockIdx.x * cgs + cg) * 8;
    const int t = col >= n ? 0 : n - col >= 8 ? 8 : (int)(n - col);
    const half8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
    float s[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    if (t > 0) {
        for (int64_t i0 = rg; i0 < batch; i0 += 8 * rgs) {
            half8_t v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                v[u] = zero;
                const int64_t i = i0 + (int64_t)u * rgs;
                if (i < batch) {
                    const half_t* src = grad_out + i * n + col;
                    v[u] = t == 8 ? load_half8_any(src) : load_half8_head_any(src, t, zero);
                }
            }
#pragma unroll
            for (int u = 0; u < 8; ++u)
#pragma unroll
                for (int e = 0; e < 8; ++e) s[e] += (float)v[u][e];
        }
    }
    if (rgs > 1) {
#pragma unroll
        for (int e = 0; e < 8; ++e) red[rg * (cgs * 8) + cg * 8 + e] = s[e];
        __syncthreads();
        if (rg != 0) return;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            float a = s[e];
            for (int g = 1; g < rgs; ++g) a += red[g * (cgs * 8) + cg * 8 + e];
            s[e] = a;
        }
    }
    if (t == 0) return;
    half8_t r;
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = round_f16(s[e]);
    if (t == 8) store_half8_any(grad + col, r);
    else store_half8_head_any(grad + col, t, r);
}

// grad[i] = sum_{b, j} (WITH_X ? x[b,i,j] : 1) * grad_out[b,i,j]            cu_arith_ln_mul_backward / _ln_add_backward
template <bool WITH_X>
__global__ __launch_bounds__(256) void k_ln_backward(int64_t batch, int64_t n, int64_t m, const half_t* __restrict__ x,
                                                     const half_t* __restrict__ grad_out, half_t* __restrict__ grad, int vec) {
    __shared__ float red[4];
    const int64_t ch = blockIdx.x;
    float s = 0.0f;
    if (vec) {         // m >= 8: the (b, j) pairs of this channel in pieces of 8, at whatever address a piece starts (global
                       // loads need no alignment); the piece across a row's end in narrower loads, zeros beyond it
        const uint32_t m8 = (uint32_t)((m + 7) >> 3), db = 256u / m8, dj = 256u % m8;      // one step of 256 pieces, as rows and remainder
        const int tail = (int)(m & 7);
        const half8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
        uint32_t b = threadIdx.x / m8, j8 = threadIdx.x % m8;
        for (; b < (uint32_t)batch; b += db, j8 += dj) {
            if (j8 >= m8) {
                j8 -= m8;
                if (++b >= (uint32_t)batch) break;
            }
            const int64_t o = ((int64_t)b * n + ch) * m + ((int64_t)j8 << 3);
            const bool whole = tail == 0 || j8 + 1 < m8;
            const half8_t gv = whole ? load_half8_any(grad_out + o) : load_half8_head_any(grad_out + o, tail, zero);
            if (WITH_X) {
                const half8_t xv = whole ? load_half8_any(x + o) : load_half8_head_any(x + o, tail, zero);
#pragma unroll
                for (int e = 0; e < 8; ++e) s += (float)xv[e] * (float)gv[e];
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) s += (float)gv[e];
            }
        }
    } else {
        for (int64_t b = 0; b < batch; ++b) {
            const int64_t base = (b * n + ch) * m;
            for (int64_t j = threadIdx.x; j < m; j += 256)
                s += WITH_X ? (float)x[base + j] * (float)grad_out[base + j] : (float)grad_out[base + j];
        }
    }
    s = block_sum<4>(s, red);
    if (threadIdx.x == 0) grad[ch] = (half_t)s;
}

// ---------------------------------------------------------------------------------------
// Reductions over dim 1 of (batch, n, m) followed by an elementwise pass.  Workgroup = 64
// columns x 4 row groups; gridDim = (ceil(m/64), batch).
// ---------------------------------------------------------------------------------------
// (kColAbsmax: the column scales alone, cu_gemm_calc_scale_transpose; only the team kernel below knows it)
enum : int { kLnFwdV = 0, kLnFwdMV = 1, kLnBwdV = 2, kLnBwdMV = 3, kSoftmaxBwd = 4, kScaleRound = 5, kColAbsmax = 6 };

struct ColArgs {
    int32_t n, m;
    const half_t* a;       // mat / out (softmax)
    const half_t* g;       // grad_in (backward kinds)
    const half_t* mean;    // (batch, m)
    const half_t* var;     // (batch, m)  (reciprocal standard deviation, as the forward kernels write it)
    const half_t* sx;      // row scales for kScaleRound
    half_t* out;           // elementwise result (fp16 kinds)
    int8_t* out_i8;        // kScaleRound
    half_t* out_mean;
    half_t* out_var;       // also scale_y for kScaleRound
    float eps;
    int bc;                // kScaleRound: row scales shared by the batch
};

template <int KIND>
__global__ __launch_bounds__(256) void k_col(ColArgs p) {
    __shared__ float red[2][4][64];
    __shared__ float tot[2][64];
    const int c = threadIdx.x & 63, rg = threadIdx.x >> 6;      // 64 columns x 4 row groups
    const int32_t col = blockIdx.x * 64 + c;
    const int64_t b = blockIdx.y;
    const int64_t boff = b * p.n * p.m;
    const bool live = col < p.m;
    float mean = 0.0f, var = 0.0f;
    if (live && (KIND == kLnBwdV || KIND == kLnBwdMV)) var = (float)p.var[b * p.m + col];
    if (live && KIND == kLnBwdMV) mean = (float)p.mean[b * p.m + col];
    const float c3 = -0.5f * var * var * var;
    float s0 = 0.0f, s1 = 0.0f;
    if (live) {
        for (int32_t i = rg; i < p.n; i += 4) {
            const int64_t o = boff + (int64_t)i * p.m + col;
            const float x = (float)p.a[o];
            if (KIND == kLnFwdV) s1 += x * x;
            else if (KIND == kLnFwdMV) { s0 += x; s1 += x * x; }
            else if (KIND == kLnBwdV) s0 += (float)p.g[o] * c3 * x;
            else if (KIND == kLnBwdMV) { const float gi = (float)p.g[o]; s0 += gi * c3 * (x - mean); s1 += -gi * var; }
            else if (KIND == kSoftmaxBwd) s0 += x * (float)p.g[o];
            else s0 = fmaxf(s0, fabsf(x * (float)p.sx[(p.bc ? 0 : b * p.n) + i]));
        }
    }
    red[0][rg][c] = s0;
    red[1][rg][c] = s1;
    __syncthreads();
    if (rg == 0) {
        if (KIND == kScaleRound) tot[0][c] = fmaxf(fmaxf(red[0][0][c], red[0][1][c]), fmaxf(red[0][2][c], red[0][3][c]));
        else tot[0][c] = red[0][0][c] + red[0][1][c] + red[0][2][c] + red[0][3][c];
        tot[1][c] = red[1][0][c] + red[1][1][c] + red[1][2][c] + red[1][3][c];
    }
    __syncthreads();
    s0 = tot[0][c];
    s1 = tot[1][c];
    if (!live) return;
    const float fn = (float)p.n;
    float k0 = 0.0f, k1 = 0.0f;        // per-column constants of the elementwise pass
    if (KIND == kLnFwdV) {
        k1 = rsqrtf(s1 / fn + p.eps);
        if (rg == 0) p.out_var[b * p.m + col] = (half_t)k1;
    } else if (KIND == kLnFwdMV) {
        k0 = s0 / fn;
        k1 = rsqrtf(s1 / fn - k0 * k0 + p.eps);
        if (rg == 0) { p.out_var[b * p.m + col] = (half_t)k1; p.out_mean[b * p.m + col] = (half_t)k0; }
    } else if (KIND == kLnBwdMV) {
        s1 -= 2.0f * s0 * mean;        // local_grad_mean -= 2 * local_grad_var * local_mean
    } else if (KIND == kScaleRound) {
        k0 = (float)((double)s0 / 127.0);        // float / double constant, as the reference writes it
        if (rg == 0) p.out_var[b * p.m + col] = (half_t)k0;
    }
    for (int32_t i = rg; i < p.n; i += 4) {
        const int64_t o = boff + (int64_t)i * p.m + col;
        const float x = (float)p.a[o];
        if (KIND == kLnFwdV) p.out[o] = round_f16(x * k1);
        else if (KIND == kLnFwdMV) p.out[o] = round_f16((x - k0) * k1);
        else if (KIND == kLnBwdV) p.out[o] = round_f16((float)p.g[o] * var + (s0 * x * 2.0f) / fn);
        else if (KIND == kLnBwdMV) p.out[o] = round_f16((float)p.g[o] * var + (s1 + s0 * x * 2.0f) / fn);
        else if (KIND == kSoftmaxBwd) p.out[o] = round_f16(x * ((float)p.g[o] - s0));
        else p.out_i8[o] = (int8_t)quant_i8(x * (float)p.sx[(p.bc ? 0 : b * p.n) + i], k0);
    }
}

// The same reductions with the tile in registers: 64 columns x 512 rows per workgroup (16-byte
// loads, each input read once), taller columns shared by a team of up to 32 workgroups that
// exchange their partial column statistics (exchange.h).  Used when the shape allows 16-byte
// accesses; k_col above serves everything else.
constexpr int kColTeamMaxParts = 32;

// MODE 0: 16-byte accesses with the non-temporal hint (the tile's row segments are whole cache lines: m % 64 == 0, buffers on
// 128-byte boundaries); 1: 16-byte accesses without it; 2: any m and alignment (pieces inside a row still whole, at whatever
// address they lie; the piece across a row's end in at most three narrower accesses).
template <int KIND, int MODE>
__global__ __launch_bounds__(512) void k_col_team(ColArgs p, int32_t tiles_per_batch, int32_t parts, uint32_t nteams, XchLaunch xl) {
    uint64_t* const xch = xl.region;
    const uint32_t tag = xl.tag;
    constexpr int NT = 512, LPR = 8, R = 8;
    using T = ColTile<NT, LPR, R>;
    constexpr bool TWO = KIND != kLnFwdV && KIND != kLnFwdMV && KIND != kScaleRound && KIND != kColAbsmax;     // reads grad_in too
    constexpr bool IS_MAX = KIND == kScaleRound || KIND == kColAbsmax;
    constexpr int NV = (KIND == kLnFwdMV || KIND == kLnBwdMV) ? 2 : 1;      // statistics per column
    __shared__ float lds[(T::NW + 1) * T::COLS * NV];
    __shared__ float tot[T::COLS * 2];
    const int tid = threadIdx.x, cg = tid % LPR, rg = tid / LPR;
    XchMember me;
    if (!xch_member(blockIdx.x, parts, nteams, me)) return;
    const uint32_t part = me.part, team = me.team;
    const uint32_t b = team / tiles_per_batch, ct = team - b * tiles_per_batch;
    const int32_t col0 = ct * T::COLS + cg * 8;
    const int32_t own0 = part * T::ROWS;
    const int32_t own_n = min(T::ROWS, p.n - own0);
    const int64_t boff = (int64_t)b * p.n * p.m + (int64_t)own0 * p.m;
    const bool live = col0 < p.m;

    // The per-column and per-row operands of the sums are requested ahead of the tiles: loads return in
    // order, and behind the tiles they would hold the sums back until the last piece had arrived.
    half8_t hv = {0, 0, 0, 0, 0, 0, 0, 0}, hm = {0, 0, 0, 0, 0, 0, 0, 0};
    half_t sxh[R];
    constexpr bool NTH = MODE == 0, UA = MODE == 2;
    auto load8 = [&](const half_t* src) __attribute__((always_inline)) {       // eight per-column values of this lane's columns
        half8_t r = {0, 0, 0, 0, 0, 0, 0, 0};
        if constexpr (UA) {
            if (col0 + 8 <= p.m) r = load_half8_any(src);
            else if (col0 < p.m) r = load_half8_head_any(src, p.m & 7, r);
        } else {
            r = *reinterpret_cast<const half8_t*>(src);
        }
        return r;
    };
    auto store8 = [&](half_t* dst, half8_t r) __attribute__((always_inline)) {
        if constexpr (UA) {
            if (col0 + 8 <= p.m) store_half8_any(dst, r);
            else if (col0 < p.m) store_half8_head_any(dst, p.m & 7, r);
        } else {
            *reinterpret_cast<half8_t*>(dst) = r;
        }
    };
    if (live && (KIND == kLnBwdV || KIND == kLnBwdMV)) hv = load8(p.var + (int64_t)b * p.m + col0);
    if (live && KIND == kLnBwdMV) hm = load8(p.mean + (int64_t)b * p.m + col0);
#pragma unroll
    for (int q = 0; q < R; ++q) {
        sxh[q] = (half_t)0.0f;
        if (KIND == kScaleRound) {
            const int32_t row = own0 + q * T::RPP + rg;
            if (row < p.n) sxh[q] = p.sx[(p.bc ? 0 : (int64_t)b * p.n) + row];
        }
    }
    half8_t va[R], vg[TWO ? R : 1];
    // every input byte is read once: non-temporal loads; non-temporal stores too, except for the softmax
    // gradient, where they measured 1-2 % slower
    constexpr bool NTS = NTH && KIND != kSoftmaxBwd;
    coltile_load<NT, LPR, R, NTH, UA>(va, p.a + boff, own_n, p.m, col0, (half_t)0.0f);
    if constexpr (TWO) coltile_load<NT, LPR, R, NTH, UA>(vg, p.g + boff, own_n, p.m, col0, (half_t)0.0f);
    float mean[8], var[8], c3[8], sxv[R];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        var[e] = (float)hv[e];
        c3[e] = -0.5f * var[e] * var[e] * var[e];
        mean[e] = (float)hm[e];
    }
#pragma unroll
    for (int q = 0; q < R; ++q) sxv[q] = (float)sxh[q];

    float s[NV * 8];
#pragma unroll
    for (int e = 0; e < NV * 8; ++e) s[e] = 0.0f;
#pragma unroll
    for (int q = 0; q < R; ++q)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float x = (float)va[q][e];
            const float gi = TWO ? (float)vg[TWO ? q : 0][e] : 0.0f;
            if constexpr (KIND == kLnFwdV) s[e] += x * x;
            else if constexpr (KIND == kLnFwdMV) { s[e] += x; s[8 + e] += x * x; }
            else if constexpr (KIND == kLnBwdV) s[e] += gi * c3[e] * x;
            else if constexpr (KIND == kLnBwdMV) { s[e] += gi * c3[e] * (x - mean[e]); s[8 + e] += -gi * var[e]; }
            else if constexpr (KIND == kSoftmaxBwd) s[e] += x * gi;
            else if constexpr (KIND == kColAbsmax) s[e] = fmaxf(s[e], fabsf(x));
            else s[e] = fmaxf(s[e], fabsf(x * sxv[q]));
        }
    if (parts == 1) {
        coltile_reduce<NT, LPR, NV, IS_MAX>(s, lds);      // every lane: the statistics of its 8 columns
    } else {
        uint64_t* team_slots = xch + (size_t)team * parts * kXchVals;
        // this part's statistics go straight from the reduction to its slot
        coltile_reduce_to<NT, LPR, NV, IS_MAX>(s, lds, [&](int i, float r) { xch_post(team_slots + (size_t)part * kXchVals, i, r, tag); });
        if (tid < T::COLS * NV) {
            const uint64_t deadline = wall_clock64() + kXchTimeoutTicks;
            float acc = 0.0f;
            bool ok = true;
            // four parts per round trip: eight would push the kernels that can stay within 128 registers (two workgroups
            // per compute unit) beyond them
            for (int32_t q0 = 0; q0 < parts; q0 += 4) {
                float x[4];
                ok &= xch_gather<4>(team_slots, parts, q0, tid, tag, deadline, x);
#pragma unroll
                for (int j = 0; j < 4; ++j) acc = IS_MAX ? fmaxf(acc, x[j]) : acc + x[j];     // part order; absent parts are zeros
            }
            tot[tid] = ok ? acc : __builtin_nanf("");
            if (!ok) xch_flag(xl, kXchStatusTimeout);
        }
        __syncthreads();
#pragma unroll
        for (int e = 0; e < NV * 8; ++e) s[e] = tot[(e >> 3) * T::COLS + cg * 8 + (e & 7)];
    }

    const float fn = (float)p.n;
    float k0[8], k1[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        k0[e] = k1[e] = 0.0f;
        if constexpr (KIND == kLnFwdV) k1[e] = rsqrtf(s[e] / fn + p.eps);
        else if constexpr (KIND == kLnFwdMV) { k0[e] = s[e] / fn; k1[e] = rsqrtf(s[8 + e] / fn - k0[e] * k0[e] + p.eps); }
        else if constexpr (KIND == kLnBwdMV) s[8 + e] -= 2.0f * s[e] * mean[e];        // local_grad_mean -= 2 * local_grad_var * local_mean
        else if constexpr (KIND == kScaleRound) k0[e] = (float)((double)s[e] / 127.0);     // float / double constant, as the reference writes it
    }
    if (live && part == 0 && rg == 0) {
        half8_t h0, h1;
#pragma unroll
        for (int e = 0; e < 8; ++e) { h0[e] = (half_t)k0[e]; h1[e] = (half_t)k1[e]; }
        if (KIND == kLnFwdV || KIND == kLnFwdMV) store8(p.out_var + (int64_t)b * p.m + col0, h1);
        if (KIND == kLnFwdMV) store8(p.out_mean + (int64_t)b * p.m + col0, h0);
        if (KIND == kScaleRound) store8(p.out_var + (int64_t)b * p.m + col0, h0);
        if constexpr (KIND == kColAbsmax) {
#pragma unroll
            for (int e = 0; e < 8; ++e) h0[e] = scale_from_absmax(s[e]);
            store8(p.out_var + (int64_t)b * p.m + col0, h0);
        }
    }
    if constexpr (KIND == kColAbsmax) {
        // the scales are all there is to write
    } else if constexpr (KIND == kScaleRound) {
        if (live) {
#pragma unroll
            for (int q = 0; q < R; ++q) {
                const int32_t lrow = q * T::RPP + rg;
                if (lrow < own_n) {
                    int32_t t[8];
#pragma unroll
                    for (int e = 0; e < 8; ++e) t[e] = quant_i8((float)va[q][e] * sxv[q], k0[e]);
                    int8_t* dst = p.out_i8 + boff + ((uint32_t)lrow * (uint32_t)p.m + (uint32_t)col0);
                    if constexpr (UA) {
                        if (col0 + 8 <= p.m) {
                            store_byte8_any(dst, pack4_i8(t[0], t[1], t[2], t[3]), pack4_i8(t[4], t[5], t[6], t[7]));
                        } else {
                            store_byte8_head_any(dst, p.m & 7, pack4_i8(t[0], t[1], t[2], t[3]), pack4_i8(t[4], t[5], t[6], t[7]));
                        }
                    } else {
                        *reinterpret_cast<uint2_t*>(dst) = uint2_t{pack4_i8(t[0], t[1], t[2], t[3]), pack4_i8(t[4], t[5], t[6], t[7])};
                    }
                }
            }
        }
    } else {
#pragma unroll
        for (int q = 0; q < R; ++q)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float x = (float)va[q][e];
                const float gi = TWO ? (float)vg[TWO ? q : 0][e] : 0.0f;
                float o;
                if constexpr (KIND == kLnFwdV) o = x * k1[e];
                else if constexpr (KIND == kLnFwdMV) o = (x - k0[e]) * k1[e];
                else if constexpr (KIND == kLnBwdV) o = gi * var[e] + (s[e] * x * 2.0f) / fn;
                else if constexpr (KIND == kLnBwdMV) o = gi * var[e] + (s[8 + e] + s[e] * x * 2.0f) / fn;
                else o = x * (gi - s[e]);
                va[q][e] = round_f16(o);
            }
        coltile_store<NT, LPR, R, NTS, UA>(va, p.out + boff, own_n, p.m, col0);
    }
    if (parts > 1 && tid < 64) xch_retire(xl, team, parts);
}

// cu_gemm_backward_round_scale: per-row absmax of mat * scale_y[col] -> scale_x, then rounding.
__global__ __launch_bounds__(256) void k_round_scale_rows(int32_t n, int32_t m, const half_t* __restrict__ mat,
                                                          const half_t* __restrict__ scale_y, int8_t* __restrict__ out,
                                                          half_t* __restrict__ scale_x, int bc) {
    __shared__ float red[4];
    const int64_t row = blockIdx.x;                    // b*n + i
    const int64_t b = row / n;
    const half_t* x = mat + row * m;
    const half_t* sy = scale_y + (bc ? 0 : b * m);
    float mx = 0.0f;
    for (int32_t j = threadIdx.x; j < m; j += 256) mx = fmaxf(fabsf((float)x[j] * (float)sy[j]), mx);
    mx = block_max<4>(mx, red);
    const float s = (float)((double)mx / 127.0);
    if (threadIdx.x == 0) scale_x[row] = (half_t)s;
    for (int32_t j = threadIdx.x; j < m; j += 256) out[row * m + j] = (int8_t)quant_i8((float)x[j] * (float)sy[j], s);
}

// The same with a wave per row and 16-byte accesses (m % 8 == 0, aligned pointers); the second pass
// over the row finds it in the cache.
__global__ __launch_bounds__(256) void k_round_scale_rows_wide(int64_t rows, int32_t n, int32_t m, const half_t* __restrict__ mat,
                                                               const half_t* __restrict__ scale_y, int8_t* __restrict__ out,
                                                               half_t* __restrict__ scale_x, int bc) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int64_t b = row / n;
    const half_t* x = mat + row * m;
    const half_t* sy = scale_y + (bc ? 0 : b * m);
    float mx = 0.0f;
    for (int32_t j = lane * 8; j < m; j += 512) {
        const half8_t xv = *reinterpret_cast<const half8_t*>(x + j), sv = *reinterpret_cast<const half8_t*>(sy + j);
#pragma unroll
        for (int e = 0; e < 8; ++e) mx = fmaxf(fabsf((float)xv[e] * (float)sv[e]), mx);
    }
    mx = wave_max(mx);
    const float s = (float)((double)mx / 127.0);
    if (lane == 0) scale_x[row] = (half_t)s;
    for (int32_t j = lane * 8; j < m; j += 512) {
        const half8_t xv = *reinterpret_cast<const half8_t*>(x + j), sv = *reinterpret_cast<const half8_t*>(sy + j);
        int32_t t[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) t[e] = quant_i8((float)xv[e] * (float)sv[e], s);
        *reinterpret_cast<uint2_t*>(out + row * m + j) = uint2_t{pack4_i8(t[0], t[1], t[2], t[3]), pack4_i8(t[4], t[5], t[6], t[7])};
    }
}

// The same for rows of at most 2048 columns, kept in registers: a wave takes U consecutive rows of P 16-byte pieces
// per lane (P * U = 4 loads in flight per lane, the matrix read once and with the non-temporal hint), finds each
// row's maximum over the wave with data-parallel-primitive operands and rounds from the registers.
// UA: rows that are not whole 16-byte pieces or buffers off 16-byte boundaries -- a piece inside its row still comes in
// one 16-byte load and leaves in one 8-byte store (global accesses need no alignment), the piece across a row's end
// in at most three narrower accesses each way.
template <int P, int U, bool UA>
__global__ __launch_bounds__(256) void k_round_scale_rows_reg(int64_t rows, int32_t n, int32_t m, const half_t* __restrict__ mat,
                                                              const half_t* __restrict__ scale_y, int8_t* __restrict__ out,
                                                              half_t* __restrict__ scale_x, int bc) {
    const int lane = threadIdx.x & 63;
    const int64_t row0 = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * U;
    if (row0 >= rows) return;
    auto load8 = [&](const half_t* src, int32_t j, bool nt) __attribute__((always_inline)) {
        half8_t r = {0, 0, 0, 0, 0, 0, 0, 0};
        if constexpr (!UA) {
            r = nt ? __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(src + j)) : *reinterpret_cast<const half8_t*>(src + j);
        } else if (j + 8 <= m) {
            r = load_half8_any(src + j);
        } else {
            r = load_half8_head_any(src + j, m & 7, r);       // (callers pass j < m)
        }
        return r;
    };
    half8_t xv[U][P], sv[U][P];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int64_t row = row0 + u < rows ? row0 + u : rows - 1;
        const half_t* x = mat + row * m;
        const half_t* sy = scale_y + (bc ? 0 : (row / n) * m);
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const int32_t j = lane * 8 + p * 512;
            xv[u][p] = sv[u][p] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
            if (j < m) {
                xv[u][p] = load8(x, j, true);
                sv[u][p] = load8(sy, j, false);
            }
        }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        float mx = 0.0f;
#pragma unroll
        for (int p = 0; p < P; ++p)
#pragma unroll
            for (int e = 0; e < 8; ++e) mx = fmaxf(fabsf((float)xv[u][p][e] * (float)sv[u][p][e]), mx);
        mx = __builtin_bit_cast(float, wave_max_u32_uniform(__builtin_bit_cast(uint32_t, mx)));      // (non-negative floats order as their bits)
        const float s = (float)((double)mx / 127.0);
        const int64_t row = row0 + u;
        if (row < rows) {
            if (lane == 0) scale_x[row] = (half_t)s;
#pragma unroll
            for (int p = 0; p < P; ++p) {
                const int32_t j = lane * 8 + p * 512;
                if (j < m) {
                    int32_t t[8];
#pragma unroll
                    for (int e = 0; e < 8; ++e) t[e] = quant_i8((float)xv[u][p][e] * (float)sv[u][p][e], s);
                    int8_t* dst = out + row * m + j;
                    if constexpr (!UA) {
                        *reinterpret_cast<uint2_t*>(dst) = uint2_t{pack4_i8(t[0], t[1], t[2], t[3]), pack4_i8(t[4], t[5], t[6], t[7])};
                    } else if (j + 8 <= m) {
                        store_byte8_any(dst, pack4_i8(t[0], t[1], t[2], t[3]), pack4_i8(t[4], t[5], t[6], t[7]));
                    } else {
                        store_byte8_head_any(dst, m & 7, pack4_i8(t[0], t[1], t[2], t[3]), pack4_i8(t[4], t[5], t[6], t[7]));
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------
// Gradient of the relative-position bias: grad[h, bucket] = sum of grad_out[h, k, q] over the
// (k, q) that map to the bucket.  One workgroup per head, a bucket histogram in LDS.
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_position_backward(int32_t query_len, int32_t key_len, int32_t num_buckets,
                                                           int32_t max_distance, const int32_t* __restrict__ mapping,
                                                           const half_t* __restrict__ grad_out, half_t* __restrict__ grad,
                                                           int bidirectional) {
    extern __shared__ float hist[];
    const int h = blockIdx.x;
    for (int i = threadIdx.x; i < num_buckets; i += 256) hist[i] = 0.0f;
    __syncthreads();
    const int64_t total = (int64_t)key_len * query_len;
    const half_t* g = grad_out + (int64_t)h * total;
    for (int64_t i = threadIdx.x; i < total; i += 256) {
        int32_t rel = (int32_t)(i % query_len) - (int32_t)(i / query_len);
        int32_t off = 0;
        if (rel < 0) {
            if (bidirectional) { rel = -rel; off = num_buckets / 2; }
            else rel = 0;
        }
        if (rel >= max_distance) rel = max_distance - 1;
        atomicAdd(&hist[mapping[rel] + off], (float)g[i]);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < num_buckets; i += 256) grad[(int64_t)h * num_buckets + i] = (half_t)hist[i];
}

// The same with the key rows of a head split over a team of workgroups (exchange.h; at most 128
// buckets, the packets of one slot).  A thread walks down a column q of its rows: rel = q - k
// falls by one per row, so the bucket changes rarely and the thread adds a whole run to the LDS
// histogram at once.  Part 0 collects the partial histograms in part order and writes the result.
__global__ __launch_bounds__(256) void k_position_backward_team(int32_t query_len, int32_t key_len, int32_t num_buckets,
                                                                int32_t max_distance, const int32_t* __restrict__ mapping,
                                                                const half_t* __restrict__ grad_out, half_t* __restrict__ grad,
                                                                int bidirectional, int32_t parts, int32_t rows_per_part,
                                                                uint32_t nteams, XchLaunch xl) {
    uint64_t* const xch = xl.region;
    const uint32_t tag = xl.tag;
    extern __shared__ float hist[];                       // num_buckets floats, then max_distance bucket numbers
    int32_t* lmap = reinterpret_cast<int32_t*>(hist + num_buckets);
    XchMember me;                                          // a head's parts are a team
    if (!xch_member(blockIdx.x, parts, nteams, me)) return;
    const uint32_t part = me.part, h = me.team;
    const int tid = threadIdx.x;
    for (int i = tid; i < num_buckets; i += 256) hist[i] = 0.0f;
    for (int i = tid; i < max_distance; i += 256) lmap[i] = mapping[i];
    __syncthreads();
    const int32_t k0 = part * rows_per_part, k1 = min(key_len, k0 + rows_per_part);
    const half_t* g = grad_out + (int64_t)h * key_len * query_len;
    const int32_t half_b = num_buckets / 2;
    for (int32_t q = tid; q < query_len; q += 256) {
        float run = 0.0f;
        int32_t cur = -1;
        for (int32_t k = k0; k < k1; ++k) {
            int32_t rel = q - k, off = 0;
            if (rel < 0) {
                if (bidirectional) { rel = -rel; off = half_b; }
                else rel = 0;
            }
            if (rel >= max_distance) rel = max_distance - 1;
            const int32_t bucket = lmap[rel] + off;
            const float v = (float)g[(int64_t)k * query_len + q];
            if (bucket != cur) {
                if (cur >= 0) atomicAdd(&hist[cur], run);
                cur = bucket;
                run = 0.0f;
            }
            run += v;
        }
        if (cur >= 0) atomicAdd(&hist[cur], run);
    }
    __syncthreads();
    if (parts == 1) {
        for (int i = tid; i < num_buckets; i += 256) grad[(int64_t)h * num_buckets + i] = (half_t)hist[i];
        return;
    }
    uint64_t* team_slots = xch + (size_t)h * parts * kXchVals;
    for (int i = tid; i < num_buckets; i += 256) xch_post(team_slots + (size_t)part * kXchVals, i, hist[i], tag);
    if (part == 0) {
        const uint64_t deadline = wall_clock64() + kXchTimeoutTicks;
        for (int i = tid; i < num_buckets; i += 256) {
            float acc = 0.0f;
            bool ok = true;
            for (int32_t p0 = 0; p0 < parts; p0 += 8) {
                float x[8];
                ok &= xch_gather<8>(team_slots, parts, p0, i, tag, deadline, x);
#pragma unroll
                for (int j = 0; j < 8; ++j) acc += x[j];
            }
            grad[(int64_t)h * num_buckets + i] = ok ? (half_t)acc : (half_t)__builtin_nanf("");
            if (!ok) xch_flag(xl, kXchStatusTimeout);
        }
        __syncthreads();
    }
    if (tid < 64) xch_retire(xl, h, parts);
}

// The same team layout for query rows of whole 16-byte pieces: the bias depends on q - k only, so the sum over
// a bucket is a sum over diagonals of grad_out.  A thread takes pieces of eight key rows x eight queries (eight
// 16-byte non-temporal loads in flight, pieces dealt query-fastest so that a wave reads whole rows), adds the 64
// values into the 15 diagonals that cross the piece -- element (row kk, query e) belongs to diagonal e - kk, a
// register chosen at compile time -- and leaves the 15 sums in the piece's place in LDS.  Then a thread per
// diagonal adds the pieces' contributions to it (two pieces per block of eight rows) in a fixed order: no
// atomics up to here.  At the end the diagonals' sums go into the bucket histogram, and the parts' histograms
// to part 0 as above.
__global__ __launch_bounds__(256) void k_position_backward_diag(int32_t query_len, int32_t key_len, int32_t num_buckets,
                                                                int32_t max_distance, const int32_t* __restrict__ mapping,
                                                                const half_t* __restrict__ grad_out, half_t* __restrict__ grad,
                                                                int bidirectional, int32_t parts, int32_t rows_per_part,
                                                                uint32_t nteams, XchLaunch xl) {
    uint64_t* const xch = xl.region;
    const uint32_t tag = xl.tag;
    extern __shared__ float psm[];
    float* hist = psm;                                    // num_buckets
    float* stage = psm + num_buckets;                     // 15 floats per piece of the part
    XchMember me;
    if (!xch_member(blockIdx.x, parts, nteams, me)) return;
    const uint32_t part = me.part, h = me.team;
    const int tid = threadIdx.x;
    const int32_t k0 = part * rows_per_part, k1 = min(key_len, k0 + rows_per_part);
    const int32_t rel_min = -(k1 - 1), nd = query_len + (k1 - k0) - 1;      // rel = q - k of the part's rows: rel_min + [0, nd)
    for (int i = tid; i < num_buckets; i += 256) hist[i] = 0.0f;
    const half_t* g = grad_out + (int64_t)h * key_len * query_len;
    const int32_t ncp = query_len >> 3, nrb = (k1 - k0 + 7) >> 3;
    for (int32_t pi = tid; pi < ncp * nrb; pi += 256) {
        const int32_t rb = pi / ncp, cp = pi - rb * ncp;
        const int32_t kr = k0 + rb * 8;
        half8_t v[8];
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) {
            const int32_t row = min(kr + kk, k1 - 1);      // (rows past the part's last repeat it and are left out below)
            v[kk] = __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(g + (int64_t)row * query_len) + cp);
        }
        float d[15];
#pragma unroll
        for (int j = 0; j < 15; ++j) d[j] = 0.0f;
#pragma unroll
        for (int kk = 0; kk < 8; ++kk)
#pragma unroll
            for (int e = 0; e < 8; ++e) d[e - kk + 7] += (kr + kk < k1) ? (float)v[kk][e] : 0.0f;
#pragma unroll
        for (int j = 0; j < 15; ++j) stage[pi * 15 + j] = d[j];       // d[j]: diagonal rel = 8 cp - kr + j - 7
    }
    __syncthreads();
    const int32_t half_b = num_buckets / 2;
    for (int32_t r = tid; r < nd; r += 256) {
        float sum = 0.0f;
        for (int32_t rb = 0; rb < nrb; ++rb) {
            const int32_t t = r + rel_min + k0 + 8 * rb + 7;          // = 8 cp + j of the pieces of this row block that hold the diagonal
            const int32_t cp = t >> 3, j = t & 7;
            if (j <= 6 && cp >= 1 && cp <= ncp) sum += stage[(rb * ncp + cp - 1) * 15 + j + 8];
            if (cp >= 0 && cp < ncp) sum += stage[(rb * ncp + cp) * 15 + j];
        }
        int32_t rel = r + rel_min, off = 0;
        if (rel < 0) {
            if (bidirectional) { rel = -rel; off = half_b; }
            else rel = 0;
        }
        if (rel >= max_distance) rel = max_distance - 1;
        atomicAdd(&hist[mapping[rel] + off], sum);
    }
    __syncthreads();
    if (parts == 1) {
        for (int i = tid; i < num_buckets; i += 256) grad[(int64_t)h * num_buckets + i] = (half_t)hist[i];
        return;
    }
    uint64_t* team_slots = xch + (size_t)h * parts * kXchVals;
    for (int i = tid; i < num_buckets; i += 256) xch_post(team_slots + (size_t)part * kXchVals, i, hist[i], tag);
    if (part == 0) {
        const uint64_t deadline = wall_clock64() + kXchTimeoutTicks;
        for (int i = tid; i < num_buckets; i += 256) {
            float acc = 0.0f;
            bool ok = true;
            for (int32_t p0 = 0; p0 < parts; p0 += 8) {
                float x[8];
                ok &= xch_gather<8>(team_slots, parts, p0, i, tag, deadline, x);
#pragma unroll
                for (int j = 0; j < 8; ++j) acc += x[j];
            }
            grad[(int64_t)h * num_buckets + i] = ok ? (half_t)acc : (half_t)__builtin_nanf("");
            if (!ok) xch_flag(xl, kXchStatusTimeout);
        }
        __syncthreads();
    }
    if (tid < 64) xch_retire(xl, h, parts);
}

// ---------------------------------------------------------------------------------------
// Embedding gradient in two stages over ids sorted per batch entry (cuda/embedding.cu:38-88):
// stage 1 sums runs of equal ids inside one batch entry, writes complete runs to grad and the
// last (possibly continuing) run to aux_grad; stage 2 adds the aux rows into grad, merging equal
// neighbours.  One thread per hidden column, sequential over the ids as in the reference, so
// sums are formed in the same order.
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_embedding_backward1(int32_t n, int32_t m, const half_t* __restrict__ grad_out,
                                                             const int32_t* __restrict__ argsort_ids,
                                                             const int32_t* __restrict__ sorted_ids, half_t* grad,
                                                             half_t* __restrict__ aux_grad, int32_t* __restrict__ aux_idx) {
    const int64_t b = blockIdx.x;
    const int32_t col = blockIdx.y * 256 + threadIdx.x;
    if (col >= m) return;
    const int64_t base = b * n;
    float sum = 0.0f;
    // eight gathers in flight at a time; the sums are still formed one id after the other
    for (int32_t i0 = 0; i0 < n; i0 += 8) {
        float v[8];
        int32_t id[9];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int32_t i = min(i0 + u, n - 1);
            v[u] = (float)grad_out[(int64_t)argsort_ids[base + i] * m + col];
            id[u] = sorted_ids[base + i];
        }
        id[8] = sorted_ids[base + min(i0 + 8, n - 1)];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int32_t i = i0 + u;
            if (i < n) {
                sum += v[u];
                if (i + 1 == n) {
                    aux_grad[b * m + col] = (half_t)sum;
                    if (col == 0) aux_idx[b] = id[u];
                } else if (id[u] != id[u + 1]) {
                    grad[(int64_t)id[u] * m + col] = (half_t)sum;
                    sum = 0.0f;
                }
            }
        }
    }
}

__global__ __launch_bounds__(256) void k_embedding_backward2(int32_t batch, int32_t m, const half_t* __restrict__ aux_grad,
                                                             const int32_t* __restrict__ aux_idx, half_t* grad) {
    const int32_t col = blockIdx.x * 256 + threadIdx.x;
    if (col >= m) return;
    float sum = 0.0f;
    for (int32_t i = 0; i < batch; ++i) {
        sum += (float)aux_grad[(int64_t)i * m + col];
        if (i + 1 == batch || aux_idx[i] != aux_idx[i + 1]) {
            half_t* gp = grad + (int64_t)aux_idx[i] * m + col;
            *gp = round_f16((float)*gp + sum);
            sum = 0.0f;
        }
    }
}

template <int OP, int BC>
static int launch_ew(int64_t rows, int64_t cols, int64_t n, const void* x, const void* a, const void* b, void* out, void* stream) {
    if (rows < 0 || cols < 0) return CPMK_EBADARG;
    if (rows * cols == 0) return 0;
    if (cols % 2) return CPMK_EALIGN;
    if (any_null(x, a, out) || ((OP == kFma || OP == kSubDiv) && b == nullptr)) return CPMK_EBADARG;
    const bool wide = cols % 8 == 0 && aligned16(x) && aligned16(out) && (BC == 2 || (aligned16(a) && (!b || aligned16(b))));
    const int64_t chunks = ceil_div(cols, 256 * 8);
    if (rows * chunks > 0x7fffffffll) return CPMK_ETOOBIG;
    const dim3 grid((unsigned)(rows * chunks));
    if (wide)
        hipLaunchKernelGGL((k_ew<OP, BC, false>), grid, dim3(256), 0, (hipStream_t)stream, cols, (uint32_t)chunks, n, (const half_t*)x,
                           (const half_t*)a, (const half_t*)b, (half_t*)out);
    else
        hipLaunchKernelGGL((k_ew<OP, BC, true>), grid, dim3(256), 0, (hipStream_t)stream, cols, (uint32_t)chunks, n, (const half_t*)x,
                           (const half_t*)a, (const half_t*)b, (half_t*)out);
    return launch_status();
}

// the arguments of batch entries b0 onwards
static ColArgs col_args_from(const ColArgs& p, int64_t b0) {
    ColArgs q = p;
    const int64_t e0 = b0 * p.n * p.m, c0 = b0 * p.m;
    q.a = p.a + e0;
    if (p.g) q.g = p.g + e0;
    if (p.out) q.out = p.out + e0;
    if (p.out_i8) q.out_i8 = p.out_i8 + e0;
    if (p.mean) q.mean = p.mean + c0;
    if (p.var) q.var = p.var + c0;
    if (p.out_mean) q.out_mean = p.out_mean + c0;
    if (p.out_var) q.out_var = p.out_var + c0;
    if (p.sx && !p.bc) q.sx = p.sx + b0 * p.n;
    return q;
}

template <int KIND>
static int launch_col(int32_t batch, const ColArgs& p, void* stream, bool missing) {
    if (batch < 0 || p.n < 0 || p.m < 0) return CPMK_EBADARG;
    if ((int64_t)batch * p.n * p.m == 0) return 0;
    if (missing) return CPMK_EBADARG;       // (a null buffer, found by the caller, in a call that has work to do)
    const int64_t tiles = ceil_div(p.m, 64), parts = ceil_div(p.n, 512);
    // 16-byte accesses when every row and buffer allows them, else the same kernel moving its columns one by one
    const bool vec16 = p.m % 8 == 0 && aligned16(p.a) && (p.g == nullptr || aligned16(p.g)) && (p.out == nullptr || aligned16(p.out)) &&
                       (p.mean == nullptr || aligned16(p.mean)) && (p.var == nullptr || aligned16(p.var)) &&
                       (p.out_mean == nullptr || aligned16(p.out_mean)) && (p.out_var == nullptr || aligned16(p.out_var)) &&
                       (p.out_i8 == nullptr || (reinterpret_cast<uintptr_t>(p.out_i8) & 7u) == 0);
    const bool wide = (int64_t)p.n * p.m < (1ll << 31) && parts <= kColTeamMaxParts && tiles * parts <= kXchSlots;
    auto on_line = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 127u) == 0; };
    const bool lines = p.m % 64 == 0 && on_line(p.a) && on_line(p.g) && on_line(p.out);      // (a null pointer counts as aligned)
    if (wide) {
        // teams use one packet slot per (team, part): batches beyond the pool go out in several launches
        const int64_t per_launch = parts > 1 ? kXchSlots / (tiles * parts) : ((1ll << 31) - 8) / (tiles * parts);
        bool no_slots = false;
        for (int64_t b0 = 0; b0 < batch; b0 += per_launch) {
            const int64_t nb = batch - b0 < per_launch ? batch - b0 : per_launch;
            const ColArgs q = col_args_from(p, b0);
            XchScope xs;
            if (parts > 1) {
                const int rc = xs.begin(tiles * nb * parts, (hipStream_t)stream);
                if (rc == kXchFull && b0 == 0) {
                    no_slots = true;       // recorded into a graph and the capture reserve is used up: the kernel without packets below
                    break;
                }
                if (rc != 0) return rc == kXchFull ? CPMK_ETOOBIG : rc;
            }
            auto go = [&](auto kern) {
                hipLaunchKernelGGL(kern, dim3((unsigned)xch_team_grid(tiles * nb, parts)), dim3(512), 0, (hipStream_t)stream, q, (int32_t)tiles,
                                   (int32_t)parts, (uint32_t)(tiles * nb), xs.xl);
            };
            if (!vec16) go(k_col_team<KIND, 2>);
            else if (lines) go(k_col_team<KIND, 0>);
            else go(k_col_team<KIND, 1>);
            const int e = launch_status();
            const int rc2 = xs.end();
            if (e != 0 || rc2 != 0) return e ? e : rc2;
        }
        if (!no_slots) return 0;
    }
    if constexpr (KIND == kColAbsmax) {
        return -1;      // (the caller has a kernel of its own for what the team kernel does not take)
    } else {
        // the batch is the grid's y dimension (at most 65535): larger batches go out in several launches
        for (int64_t b0 = 0; b0 < batch; b0 += 65535) {
            const int64_t nb = batch - b0 < 65535 ? batch - b0 : 65535;
            hipLaunchKernelGGL((k_col<KIND>), dim3((unsigned)ceil_div(p.m, 64), (unsigned)nb), dim3(256), 0, (hipStream_t)stream,
                               col_args_from(p, b0));
            if (int e = launch_status()) return e;
        }
        return 0;
    }
}

// Column scales of (batch, n, m) on the team kernel: 0, an error code, or -1 when the shape is not one it takes.
int col_absmax_team(int32_t batch, int32_t n, int32_t m, const void* mat, void* out, void* stream) {
    ColArgs p = {n, m, (const half_t*)mat, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, (half_t*)out, 0.0f, 0};
    return launch_col<kColAbsmax>(batch, p, stream, false);
}

}  // namespace cpmk

using namespace cpmk;

extern "C" {

int cpmk_arith_global_scale(int64_t n, const void* inp, float scale, void* out, void* stream) {
    clear_stale_error();
    if (n < 0) return CPMK_EBADARG;
    if (n == 0) return 0;
    if (any_null(inp, out)) return CPMK_EBADARG;
    if (n % 8 == 0 && aligned16(inp) && aligned16(out))
        hipLaunchKernelGGL((k_global_scale<8>), dim3((unsigned)ceil_div(n, 256 * 8)), dim3(256), 0, (hipStream_t)stream, n,
                           (const half_t*)inp, scale, (half_t*)out);
    else
        hipLaunchKernelGGL((k_global_scale<1>), dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, (hipStream_t)stream, n,
                           (const half_t*)inp, scale, (half_t*)out);
    return launch_status();
}
int cpmk_arith_element_mul(int32_t batch, int32_t n, const void* x, const void* y, void* out, void* stream) {
    clear_stale_error();
    if (n % 2) return CPMK_EALIGN;
    return launch_ew<kMul, 0>(1, (int64_t)batch * n, 1, x, y, nullptr, out, stream);
}
int cpmk_arith_batch_add_forward(int32_t batch, int32_t n, const void* x, const void* y, void* out, void* stream) {
    clear_stale_error();
    if (n % 2) return CPMK_EALIGN;
    return launch_ew<kAdd, 1>(batch, n, n, x, y, nullptr, out, stream);
}
int cpmk_arith_batch_mul_add(int32_t batch, int32_t n, const void* x, const void* alpha, const void* beta, void* out, void* stream) {
    clear_stale_error();
    if (n % 2) return CPMK_EALIGN;
    return launch_ew<kFma, 1>(batch, n, n, x, alpha, beta, out, stream);
}
int cpmk_arith_batch_mul(int32_t batch, int32_t n, const void* x, const void* alpha, void* out, void* stream) {
    clear_stale_error();
    if (n % 2) return CPMK_EALIGN;
    return launch_ew<kMul, 1>(batch, n, n, x, alpha, nullptr, out, stream);
}
int cpmk_arith_ln_add(int32_t batch, int32_t n, int32_t m, const void* inp, const void* beta, void* out, void* stream) {
    clear_stale_error();
    if (batch < 0 || n < 0 || m < 0) return CPMK_EBADARG;
    if (m % 2) return CPMK_EALIGN;
    return launch_ew<kAdd, 2>((int64_t)batch * n, m, n, inp, beta, nullptr, out, stream);
}
int cpmk_arith_ln_div(int32_t batch, int32_t n, int32_t m, const void* inp, const void* alpha, void* out, void* stream) {
    clear_stale_error();
    if (batch < 0 || n < 0 || m < 0) return CPMK_EBADARG;
    if (m % 2) return CPMK_EALIGN;
    return launch_ew<kDiv, 2>((int64_t)batch * n, m, n, inp, alpha, nullptr, out, stream);
}
int cpmk_arith_ln_sub_div(int32_t batch, int32_t n, int32_t m, const void* inp, const void* alpha, const void* beta, void* out,
                          void* stream) {
    clear_stale_error();
    if (batch < 0 || n < 0 || m < 0) return CPMK_EBADARG;
    if (m % 2) return CPMK_EALIGN;
    return launch_ew<kSubDiv, 2>((int64_t)batch * n, m, n, inp, alpha, beta, out, stream);
}
int cpmk_arith_batch_add_backward(int32_t batch, int32_t n, const void* grad_out, void* grad, void* stream) {
    clear_stale_error();
    if (batch < 0 || n < 0) return CPMK_EBADARG;
    if (n == 0) return 0;
    if (grad == nullptr || (batch > 0 && grad_out == nullptr)) return CPMK_EBADARG;
    // enough lanes for the whole chip: with few columns, more row groups per workgroup
    int rgs = 1;
    while (rgs < 64 && ceil_div(n, 8) * rgs < 131072 && rgs * 2 <= batch) rgs *= 2;
    hipLaunchKernelGGL(k_batch_add_backward, dim3((unsigned)ceil_div(n, (256 / rgs) * 8)), dim3(256), 0, (hipStream_t)stream, (int64_t)batch,
                       (int64_t)n, rgs, (const half_t*)grad_out, (half_t*)grad);
    return launch_status();
}
int cpmk_arith_ln_mul_backward(int32_t batch, int32_t n, int32_t m, const void* inp, const void* grad_out, void* grad, void* stream) {
    clear_stale_error();
    if (batch < 0 || n < 0 || m < 0) return CPMK_EBADARG;
    if (n == 0) return 0;
    if (grad == nullptr || ((int64_t)batch * m > 0 && any_null(inp, grad_out))) return CPMK_EBADARG;
    hipLaunchKernelGGL((k_ln_backward<true>), dim3((unsigned)n), dim3(256), 0, (hipStream_t)stream, (int64_t)batch, (int64_t)n,
                       (int64_t)m, (const half_t*)inp, (const half_t*)grad_out, (half_t*)grad, (int)(m >= 8));
    return launch_status();
}
int cpmk_arith_ln_add_backward(int32_t batch, int32_t n, int32_t m, const void* grad_out, void* grad, void* stream) {
    clear_stale_error();
    if (batch < 0 || n < 0 || m < 0) return CPMK_EBADARG;
    if (n == 0) return 0;
    if (grad == nullptr || ((int64_t)batch * m > 0 && grad_out == nullptr)) return CPMK_EBADARG;
    hipLaunchKernelGGL((k_ln_backward<false>), dim3((unsigned)n), dim3(256), 0, (hipStream_t)stream, (int64_t)batch, (int64_t)n,
                       (int64_t)m, (const half_t*)nullptr, (const half_t*)grad_out, (half_t*)grad, (int)(m >= 8));
    return launch_status();
}

int cpmk_gelu_backward(int32_t batch, int32_t n, const void* grad_out, const void* mat, void* grad, void* stream) {
    clear_stale_error();
    if (batch < 0 || n < 0) return CPMK_EBADARG;
    const int64_t total = (int64_t)batch * n;
    if (total == 0) return 0;
    if (any_null(grad_out, mat, grad)) return CPMK_EBADARG;
    if (total % 8 == 0 && aligned16(grad_out) && aligned16(mat) && aligned16(grad))
        hipLaunchKernelGGL((k_gelu_backward<8>), dim3((unsigned)ceil_div(total / 8, 256)), dim3(256), 0, (hipStream_t)stream, total,
                           (const half_t*)grad_out, (const half_t*)mat, (half_t*)grad);
    else
        hipLaunchKernelGGL((k_gelu_backward<1>), dim3((unsigned)ceil_div(total, 256)), dim3(256), 0, (hipStream_t)stream, total,
                           (const half_t*)grad_out, (const half_t*)mat, (half_t*)grad);
    return launch_status();
}

int cpmk_layernorm_forward_v(int32_t batch, int32_t n, int32_t m, const void* mat, void* out, void* out_var, float eps, void* stream) {
    clear_stale_error();
    ColArgs p = {n, m, (const half_t*)mat, nullptr, nullptr, nullptr, nullptr, (half_t*)out, nullptr, nullptr, (half_t*)out_var, eps, 0};
    return launch_col<kLnFwdV>(batch, p, stream, any_null(mat, out, out_var));
}
int cpmk_layernorm_forward_mv(int32_t batch, int32_t n, int32_t m, const void* mat, void* out, void* out_mean, void* out_var,
                              float eps, void* stream) {
    clear_stale_error();
    ColArgs p = {n, m, (const half_t*)mat, nullptr, nullptr, nullptr, nullptr, (half_t*)out, nullptr, (half_t*)out_mean,
                 (half_t*)out_var, eps, 0};
    return launch_col<kLnFwdMV>(batch, p, stream, any_null(mat, out, out_mean, out_var));
}
int cpmk_layernorm_backward_v(int32_t batch, int32_t n, int32_t m, const void* mat, const void* grad_out, const void* var, void* grad,
                              void* stream) {
    clear_stale_error();
    ColArgs p = {n, m, (const half_t*)mat, (const half_t*)grad_out, nullptr, (const half_t*)var, nullptr, (half_t*)grad, nullptr,
                 nullptr, nullptr, 0.0f, 0};
    return launch_col<kLnBwdV>(batch, p, stream, any_null(mat, grad_out, var, grad));
}
int cpmk_layernorm_backward_mv(int32_t batch, int32_t n, int32_t m, const void* mat, const void* grad_out, const void* mean,
                               const void* var, void* grad, void* stream) {
    clear_stale_error();
    ColArgs p = {n, m, (const half_t*)mat, (const half_t*)grad_out, (const half_t*)mean, (const half_t*)var, nullptr, (half_t*)grad,
                 nullptr, nullptr, nullptr, 0.0f, 0};
    return launch_col<kLnBwdMV>(batch, p, stream, any_null(mat, grad_out, mean, var, grad));
}
int cpmk_softmax_backward(int32_t batch, int32_t n, int32_t m, const void* out, const void* grad_out, void* grad, void* stream) {
    clear_stale_error();
    ColArgs p = {n, m, (const half_t*)out, (const half_t*)grad_out, nullptr, nullptr, nullptr, (half_t*)grad, nullptr, nullptr, nullptr,
                 0.0f, 0};
    return launch_col<kSoftmaxBwd>(batch, p, stream, any_null(out, grad_out, grad));
}
int cpmk_gemm_backward_scale_round(int32_t batch, int32_t n, int32_t m, const void* mat, const void* scale_x, void* out, void* scale_y,
                                   int broad_cast_x, void* stream) {
    clear_stale_error();
    ColArgs p = {n, m, (const half_t*)mat, nullptr, nullptr, nullptr, (const half_t*)scale_x, nullptr, (int8_t*)out, nullptr,
                 (half_t*)scale_y, 0.0f, broad_cast_x};
    return launch_col<kScaleRound>(batch, p, stream, any_null(mat, scale_x, out, scale_y));
}
int cpmk_gemm_backward_round_scale(int32_t batch, int32_t n, int32_t m, const void* mat, const void* scale_y, void* out, void* scale_x,
                                   int broad_cast_y, void* stream) {
    clear_stale_error();
    if (batch < 0 || n < 0 || m < 0) return CPMK_EBADARG;
    const int64_t rows = (int64_t)batch * n;
    if (rows == 0) return 0;
    if (rows > 0x7fffffff) return CPMK_ETOOBIG;
    if (scale_x == nullptr || (m > 0 && any_null(mat, scale_y, out))) return CPMK_EBADARG;
    const bool vec16 = m % 8 == 0 && aligned16(mat) && aligned16(scale_y) && (reinterpret_cast<uintptr_t>(out) & 7u) == 0;
    if (m > 0 && m <= 2048) {      // rows that a wave holds in registers
        auto go = [&](auto pc, auto uc) {
            constexpr int P = decltype(pc)::value, U = decltype(uc)::value;
            auto run = [&](auto kern) {
                hipLaunchKernelGGL(kern, dim3((unsigned)ceil_div(rows, 4 * U)), dim3(256), 0, (hipStream_t)stream, rows, n, m, (const half_t*)mat,
                                   (const half_t*)scale_y, (int8_t*)out, (half_t*)scale_x, broad_cast_y);
            };
            if (vec16) run(k_round_scale_rows_reg<P, U, false>);
            else run(k_round_scale_rows_reg<P, U, true>);
        };
        if (m <= 512) go(std::integral_constant<int, 1>{}, std::integral_constant<int, 4>{});
        else if (m <= 1024) go(std::integral_constant<int, 2>{}, std::integral_constant<int, 2>{});
        else go(std::integral_constant<int, 4>{}, std::integral_constant<int, 1>{});
        return launch_status();
    }
    if (vec16) {
        hipLaunchKernelGGL(k_round_scale_rows_wide, dim3((unsigned)ceil_div(rows, 4)), dim3(256), 0, (hipStream_t)stream, rows, n, m,
                           (const half_t*)mat, (const half_t*)scale_y, (int8_t*)out, (half_t*)scale_x, broad_cast_y);
        return launch_status();
    }
    hipLaunchKernelGGL(k_round_scale_rows, dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream, n, m, (const half_t*)mat,
                       (const half_t*)scale_y, (int8_t*)out, (half_t*)scale_x, broad_cast_y);
    return launch_status();
}

int cpmk_position_embedding_backward(int32_t query_len, int32_t key_len, int32_t num_buckets, int32_t max_distance, int32_t num_heads,
                                     const void* position_mapping, const void* grad_out, void* grad, int bidirectional, void* stream) {
    clear_stale_error();
    if (query_len < 0 || key_len < 0 || num_buckets <= 0 || max_distance <= 0 || num_heads < 0) return CPMK_EBADARG;
    if (num_heads == 0) return 0;
    if (num_buckets > 8192) return CPMK_ETOOBIG;
    if (grad == nullptr || ((int64_t)query_len * key_len > 0 && any_null(position_mapping, grad_out))) return CPMK_EBADARG;
    if (num_buckets <= kXchVals && max_distance <= 8192 && key_len > 64) {
        // key rows of a head over a team: 64 rows a part, more when that would make more than 32 parts
        int64_t rpp = 64;
        while (ceil_div(key_len, rpp) > kColTeamMaxParts) rpp *= 2;
        const int64_t parts = ceil_div(key_len, rpp);
        if ((int64_t)num_heads * parts <= kXchSlots) {
            XchScope xs;
            const int rc = xs.begin((int64_t)num_heads * parts, (hipStream_t)stream);
            if (rc != 0 && rc != kXchFull) return rc;
            const int64_t pieces = (query_len / 8) * ceil_div(rpp, 8);          // of eight key rows x eight queries, 15 floats each
            const size_t smem = (size_t)(num_buckets + pieces * 15) * sizeof(float);
            if (rc == 0 && query_len % 8 == 0 && smem <= 64 * 1024 && aligned16(grad_out)) {
                hipLaunchKernelGGL(k_position_backward_diag, dim3((unsigned)xch_team_grid(num_heads, parts)), dim3(256), smem,
                                   (hipStream_t)stream, query_len, key_len, num_buckets, max_distance, (const int32_t*)position_mapping,
                                   (const half_t*)grad_out, (half_t*)grad, bidirectional, (int32_t)parts, (int32_t)rpp,
                                   (uint32_t)num_heads, xs.xl);
                const int e = launch_status();
                const int rc2 = xs.end();
                return e ? e : rc2;
            }
            if (rc == 0) {      // (kXchFull: recorded into a graph and the capture reserve is used up: the kernel without packets below)
                hipLaunchKernelGGL(k_position_backward_team, dim3((unsigned)xch_team_grid(num_heads, parts)), dim3(256),
                                   num_buckets * sizeof(float) + max_distance * sizeof(int32_t), (hipStream_t)stream, query_len, key_len,
                                   num_buckets, max_distance, (const int32_t*)position_mapping, (const half_t*)grad_out, (half_t*)grad,
                                   bidirectional, (int32_t)parts, (int32_t)rpp, (uint32_t)num_heads, xs.xl);
                const int e = launch_status();
                const int rc2 = xs.end();
                return e ? e : rc2;
            }
        }
    }
    hipLaunchKernelGGL(k_position_backward, dim3((unsigned)num_heads), dim3(256), num_buckets * sizeof(float), (hipStream_t)stream,
                       query_len, key_len, num_buckets, max_distance, (const int32_t*)position_mapping, (const half_t*)grad_out,
                       (half_t*)grad, bidirectional);
    return launch_status();
}

int cpmk_embedding_backward_stage1(int32_t batch, int32_t seq_len, int32_t hidden_size, const void* grad_out, const void* argsort_ids,
                                   const void* sorted_ids, void* grad, void* aux_grad, void* aux_grad_idx, void* stream) {
    clear_stale_error();
    if (batch < 0 || seq_len < 0 || hidden_size < 0) return CPMK_EBADARG;
    if ((int64_t)batch * seq_len * hidden_size == 0) return 0;
    if (ceil_div(hidden_size, 256) > 65535) return CPMK_ETOOBIG;
    if (any_null(grad_out, argsort_ids, sorted_ids, grad, aux_grad, aux_grad_idx)) return CPMK_EBADARG;
    hipLaunchKernelGGL(k_embedding_backward1, dim3((unsigned)batch, (unsigned)ceil_div(hidden_size, 256)), dim3(256), 0,
                       (hipStream_t)stream, seq_len, hidden_size, (const half_t*)grad_out, (const int32_t*)argsort_ids,
                       (const int32_t*)sorted_ids, (half_t*)grad, (half_t*)aux_grad, (int32_t*)aux_grad_idx);
    return launch_status();
}
int cpmk_embedding_backward_stage2(int32_t batch, int32_t hidden_size, const void* aux_grad, const void* aux_grad_idx, void* grad,
                                   void* stream) {
    clear_stale_error();
    if (batch < 0 || hidden_size < 0) return CPMK_EBADARG;
    if ((int64_t)batch * hidden_size == 0) return 0;
    if (any_null(aux_grad, aux_grad_idx, grad)) return CPMK_EBADARG;
    hipLaunchKernelGGL(k_embedding_backward2, dim3((unsigned)ceil_div(hidden_size, 256)), dim3(256), 0, (hipStream_t)stream, batch,
                       hidden_size, (const half_t*)aux_grad, (const int32_t*)aux_grad_idx, (half_t*)grad);
    return launch_status();
}

}  // extern "C"
