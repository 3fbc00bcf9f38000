// Row/column absmax scales, fp16 -> int8 rounding and int32 -> fp16 dequantisation.
// All of these are single-pass HBM-bound streaming kernels: 16-byte loads per lane,
// wave64 butterfly reductions, no 32-lane geometry.
// Arithmetic follows cuda/gemm.cu:6-98,176-205 and cuda/gemv.cu:26-54 of the reference.
#include "common.h"

namespace cpmk {

// ---------------------------------------------------------------------------------------
// absmax over contiguous rows: out[row] = fp16(max_j |mat[row, j]| / 127)
// TPR threads cooperate on one row (64 = one wave, 256 = whole block).
// ---------------------------------------------------------------------------------------
template <int TPR, bool VEC>
__global__ __launch_bounds__(256) void k_row_absmax(int64_t rows, int32_t m,
                                                    const half_t* __restrict__ mat,
                                                    half_t* __restrict__ out) {
    __shared__ float red[4];
    constexpr int RPB = 256 / TPR;
    const int t = threadIdx.x % TPR;
    const int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / TPR;
    float mx = 0.0f;
    if (row < rows) {
        const half_t* p = mat + row * m;
        if (VEC) {
            const half8_t* p8 = reinterpret_cast<const half8_t*>(p);
            const int m8 = m >> 3;
            for (int j = t; j < m8; j += TPR) {
                half8_t v = __builtin_nontemporal_load(p8 + j);
#pragma unroll
                for (int e = 0; e < 8; ++e) mx = fmaxf(fabsf((float)v[e]), mx);
            }
        } else {
            for (int j = t; j < m; j += TPR) mx = fmaxf(fabsf((float)p[j]), mx);
        }
    }
    if (TPR == 64) {
        mx = wave_max(mx);
    } else {
        mx = block_max<4>(mx, red);
    }
    if (t == 0 && row < rows) out[row] = scale_from_absmax(mx);
}

// ---------------------------------------------------------------------------------------
// absmax over dim 1 of (b, n, m): out[b, j] = fp16(max_i |mat[b,i,j]| / 127)
// Block = 256 threads = 32 row groups x 8 lanes; each lane owns 8 adjacent columns
// (one 16-byte load per row), the 32 row groups stride over n and are combined in LDS.
// gridDim = (ceil(m/64), batch).
// ---------------------------------------------------------------------------------------
template <bool VEC>
__global__ __launch_bounds__(256) void k_col_absmax(int32_t n, int32_t m,
                                                    const half_t* __restrict__ mat,
                                                    half_t* __restrict__ out) {
    __shared__ float red[32][65];
    const int lane8 = threadIdx.x & 7, rg = threadIdx.x >> 3;
    const int col0 = blockIdx.x * 64 + lane8 * 8;
    const half_t* base = mat + (int64_t)blockIdx.y * n * m;
    float mx[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) mx[e] = 0.0f;
    if (VEC) {
        if (col0 < m) {
            for (int i = rg; i < n; i += 32) {
                half8_t v = *reinterpret_cast<const half8_t*>(base + (int64_t)i * m + col0);
#pragma unroll
                for (int e = 0; e < 8; ++e) mx[e] = fmaxf(fabsf((float)v[e]), mx[e]);
            }
        }
    } else {
        for (int i = rg; i < n; i += 32) {
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (col0 + e < m) mx[e] = fmaxf(fabsf((float)base[(int64_t)i * m + col0 + e]), mx[e]);
        }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) red[rg][lane8 * 8 + e] = mx[e];
    __syncthreads();
    if (threadIdx.x < 64) {
        float r = 0.0f;
#pragma unroll 8
        for (int g = 0; g < 32; ++g) r = fmaxf(r, red[g][threadIdx.x]);
        const int col = blockIdx.x * 64 + threadIdx.x;
        if (col < m) out[(int64_t)blockIdx.y * m + col] = scale_from_absmax(r);
    }
}

// ---------------------------------------------------------------------------------------
// rounding: out = int8(rint(x / scale)).  MODE 0: scale per row (index = element / m),
// MODE 1: scale per (batch, column) (index = b*m + j).  W elements per thread: 16 (m % 16 == 0, 16-byte aligned
// buffers), 4 (m % 4 == 0, 8-byte aligned input and scales, 4-byte aligned output) or 1.
// ---------------------------------------------------------------------------------------
template <int MODE, int W>
__global__ __launch_bounds__(256) void k_round(int64_t total, int32_t n, int32_t m,
                                               const half_t* __restrict__ mat,
                                               const half_t* __restrict__ scale,
                                               int8_t* __restrict__ out) {
    const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if constexpr (W == 4) {
        const int64_t e0 = gid * 4;
        if (e0 >= total) return;
        const int64_t row = e0 / m;            // m % 4 == 0: the 4 elements share a row
        const half4_t a = __builtin_nontemporal_load(reinterpret_cast<const half4_t*>(mat + e0));
        int32_t q[4];
        if (MODE == 0) {
            const float sr = (float)scale[row], y = 1.0f / sr;
#pragma unroll
            for (int e = 0; e < 4; ++e) q[e] = quant_i8_rcp((float)a[e], sr, y);
        } else {
            const half4_t sv = *reinterpret_cast<const half4_t*>(scale + (row / n) * m + (e0 - row * m));
#pragma unroll
            for (int e = 0; e < 4; ++e) q[e] = quant_i8((float)a[e], (float)sv[e]);
        }
        *reinterpret_cast<uint32_t*>(out + e0) = pack4_i8(q[0], q[1], q[2], q[3]);
    } else if constexpr (W == 16) {
        const int64_t e0 = gid * 16;
        if (e0 >= total) return;
        const int64_t row = e0 / m;            // m % 16 == 0: the 16 elements share a row
        const int32_t j0 = (int32_t)(e0 - row * m);
        const half8_t* p = reinterpret_cast<const half8_t*>(mat + e0);
        half8_t a = __builtin_nontemporal_load(p), b = __builtin_nontemporal_load(p + 1);
        float s[16];
        if (MODE == 0) {
            const float sr = (float)scale[row];
#pragma unroll
            for (int e = 0; e < 16; ++e) s[e] = sr;
        } else {
            const int64_t bidx = row / n;
            const half8_t* sp = reinterpret_cast<const half8_t*>(scale + bidx * m + j0);
            half8_t s0 = sp[0], s1 = sp[1];
#pragma unroll
            for (int e = 0; e < 8; ++e) { s[e] = (float)s0[e]; s[8 + e] = (float)s1[e]; }
        }
        int32_t q[16];
        if (MODE == 0) {
            const float y = 1.0f / s[0];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                q[e] = quant_i8_rcp((float)a[e], s[0], y);
                q[8 + e] = quant_i8_rcp((float)b[e], s[0], y);
            }
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                q[e] = quant_i8((float)a[e], s[e]);
                q[8 + e] = quant_i8((float)b[e], s[8 + e]);
            }
        }
        uint4_t w;
        w.x = pack4_i8(q[0], q[1], q[2], q[3]);
        w.y = pack4_i8(q[4], q[5], q[6], q[7]);
        w.z = pack4_i8(q[8], q[9], q[10], q[11]);
        w.w = pack4_i8(q[12], q[13], q[14], q[15]);
        *reinterpret_cast<uint4_t*>(out + e0) = w;
    } else {
        if (gid >= total) return;
        const int64_t row = gid / m;
        float s;
        if (MODE == 0) s = (float)scale[row];
        else s = (float)scale[(row / n) * m + (gid - row * m)];
        out[gid] = (int8_t)quant_i8((float)mat[gid], s);
    }
}

// ---------------------------------------------------------------------------------------
// dequantisation: out = fp16((f32(acc) * sx) * sy)
// MODE 0: both scales (cu_gemm_scale), MODE 1: scale_x only, MODE 2: scale_y only.
// W elements per thread: 8 (two 16-byte loads, one 16-byte store; m % 8 == 0), 4 (m % 4 == 0, 8-byte aligned
// output and column scales) or 1.
// ---------------------------------------------------------------------------------------
template <int MODE, int W>
__global__ __launch_bounds__(256) void k_dequant(int64_t total, int32_t n, int32_t m,
                                                 const int32_t* __restrict__ mat,
                                                 const half_t* __restrict__ scale_x,
                                                 const half_t* __restrict__ scale_y,
                                                 half_t* __restrict__ out, int bcx, int bcy) {
    const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
    constexpr bool VEC = W == 8;
    const int64_t e0 = gid * W;
    if (e0 >= total) return;
    const int64_t row = e0 / m;                // = b*n + i
    const int32_t j0 = (int32_t)(e0 - row * m);
    const int64_t b = row / n;
    const int32_t i = (int32_t)(row - b * n);
    float sx = 1.0f;
    if (MODE != 2) sx = (float)scale_x[bcx ? i : row];
    const half_t* sy = (MODE != 1) ? scale_y + (bcy ? 0 : b * m) + j0 : nullptr;
    if (VEC) {
        const int4_t* p = reinterpret_cast<const int4_t*>(mat + e0);
        int4_t a0 = __builtin_nontemporal_load(p), a1 = __builtin_nontemporal_load(p + 1);
        half8_t syv;
        if (MODE != 1) syv = *reinterpret_cast<const half8_t*>(sy);
        half8_t o;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int32_t acc = e < 4 ? a0[e] : a1[e - 4];
            if (MODE == 0) o[e] = dequant(acc, sx, (float)syv[e]);
            else if (MODE == 1) o[e] = round_f16(sx * (float)acc);
            else o[e] = round_f16((float)acc * (float)syv[e]);
        }
        *reinterpret_cast<half8_t*>(out + e0) = o;
    } else if (W == 4) {
        const int4_t a0 = __builtin_nontemporal_load(reinterpret_cast<const int4_t*>(mat + e0));
        half4_t syv = {0, 0, 0, 0};
        if (MODE != 1) syv = *reinterpret_cast<const half4_t*>(sy);
        half4_t o;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (MODE == 0) o[e] = dequant(a0[e], sx, (float)syv[e]);
            else if (MODE == 1) o[e] = round_f16(sx * (float)a0[e]);
            else o[e] = round_f16((float)a0[e] * (float)syv[e]);
        }
        *reinterpret_cast<half4_t*>(out + e0) = o;
    } else {
        const int32_t acc = mat[e0];
        if (MODE == 0) out[e0] = dequant(acc, sx, (float)sy[0]);
        else if (MODE == 1) out[e0] = round_f16(sx * (float)acc);
        else out[e0] = round_f16((float)acc * (float)sy[0]);
    }
}

// ---------------------------------------------------------------------------------------
// Contiguous rows of up to 64 lanes x NV x 8 halves, one wave per row, the row in registers:
// absmax -> scale (QUANT false: cu_gemm_calc_scale) and, fused, the rounding of the same
// registers (QUANT true: calc_scale + round in one pass over HBM).  Waves stride over the rows;
// the launcher picks the wave count so that every wave gets the same number of rows when the
// row count allows.  Many resident waves, each with one row in flight, hide the memory latency
// better here than fewer waves that prefetch their next row (measured).
// ---------------------------------------------------------------------------------------
// One or two tensors with rows of the same length per launch (the two operands of a product):
// virtual row r < rows0 is row r of the first, otherwise row r - rows0 of the second.
struct RowsArgs {
    const half_t* mat0; half_t* scale0; int8_t* out0; int64_t rows0;
    const half_t* mat1; half_t* scale1; int8_t* out1; int64_t rows1;
    int32_t m;
};

// (the launcher counts on 8 resident workgroups per compute unit up to NV = 8, 4 beyond)
// UA: rows that are not whole 16-byte pieces, or buffers off 16-byte boundaries: a piece inside its row still comes in one
// 16-byte load and leaves in one 8-byte store (global accesses need no alignment), the piece across a row's end in at
// most three narrower accesses each way.
template <int NV, bool QUANT, bool UA = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(UA ? (NV <= 4 ? 8 : NV <= 8 ? 4 : 2) : (NV <= 8 ? 8 : 4)))) void k_rows(RowsArgs a) {
    const int lane = threadIdx.x & 63;
    const int64_t nw = (int64_t)gridDim.x * 4;
    const int64_t rows = a.rows0 + a.rows1;
    const int32_t m = a.m;
    int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int m8 = UA ? (m + 7) >> 3 : m >> 3;
    half8_t cur[NV];
    auto load = [&](half8_t (&v)[NV], int64_t r) __attribute__((always_inline)) {
        const half_t* mat = r < a.rows0 ? a.mat0 + r * m : a.mat1 + (r - a.rows0) * m;
        const half8_t* p8 = reinterpret_cast<const half8_t*>(mat);
        // the one piece across the row's end (piece m / 8, if m % 8 != 0) comes element by element, to the lane that owns it
        half8_t tailv = {0, 0, 0, 0, 0, 0, 0, 0};
        const int jt = m >> 3;
        if constexpr (UA) {
            if ((m & 7) != 0 && (jt & 63) == lane) tailv = load_half8_head_any(mat + jt * 8, m & 7, tailv);
        }
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int j = lane + i * 64;
#pragma unroll
            for (int e = 0; e < 8; ++e) v[i][e] = (half_t)0.0f;
            if constexpr (!UA) {
                if (j < m8) v[i] = __builtin_nontemporal_load(p8 + j);
            } else {
                if (j * 8 + 8 <= m) v[i] = load_half8_any(mat + j * 8);
                else if (j == jt) v[i] = tailv;
            }
        }
    };
    // piece j (eight int8 in w) of the output row at `orow`
    auto store = [&](int8_t* orow, int j, uint2_t w) __attribute__((always_inline)) {
        if constexpr (!UA) {
            reinterpret_cast<uint2_t*>(orow)[j] = w;
        } else if (j * 8 + 8 <= m) {
            store_byte8_any(orow + j * 8, w.x, w.y);
        } else {
            store_byte8_head_any(orow + j * 8, m & 7, w.x, w.y);       // (callers pass j < ceil(m / 8))
        }
    };
    load(cur, row);
    while (true) {
        const int64_t next = row + nw;
        // |x| maxima on the packed halves as integers, then across the wave
        ushort8_t um = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < NV; ++i) um = absbits_max(um, cur[i]);
        const uint32_t ub = wave_max_u32_uniform(absbits_max_of(um));
        float mx = (float)__builtin_bit_cast(half_t, (uint16_t)ub);
        if (ub > 0x7c00u) {      // (the same for the whole wave) a NaN in the row: the maximum that skips NaN elements
            half8_t hm;
#pragma unroll
            for (int e = 0; e < 8; ++e) hm[e] = (half_t)0.0f;
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                int4_t ci = __builtin_bit_cast(int4_t, cur[i]);
                asm volatile("" : "+v"(ci));         // nothing of this rare path is to be computed ahead of the branch
                hm = __builtin_elementwise_max(hm, __builtin_elementwise_abs(__builtin_bit_cast(half8_t, ci)));
            }
            mx = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) mx = fmaxf((float)hm[e], mx);
            mx = wave_max(mx);
        }
        const half_t sh = scale_from_absmax(mx);
        const bool second = row >= a.rows0;
        const int64_t lrow = second ? row - a.rows0 : row;
        if (lane == 0) (second ? a.scale1 : a.scale0)[lrow] = sh;
        if (QUANT) {
            const float s = (float)sh, y = 1.0f / s;
            int8_t* const orow = (second ? a.out1 : a.out0) + lrow * m;
            if (scale_is_normal(sh)) {       // (the same for the whole wave) the short rounding sequence
#pragma unroll
                for (int i = 0; i < NV; ++i) {
                    const int j = lane + i * 64;
                    uint32_t q[8];
                    int4_t ci = __builtin_bit_cast(int4_t, cur[i]);
                    asm volatile("" : "+v"(ci));     // keeps the fp32 conversions of the two paths apart (hoisted above the branch they hold NV * 8 registers)
                    const half8_t ch = __builtin_bit_cast(half8_t, ci);
#pragma unroll
                    for (int e = 0; e < 8; ++e) q[e] = quant_i8_own_scale_bits((float)ch[e], s, y);
                    uint2_t w;
                    w.x = pack4_i8((int32_t)q[0], (int32_t)q[1], (int32_t)q[2], (int32_t)q[3]);
                    w.y = pack4_i8((int32_t)q[4], (int32_t)q[5], (int32_t)q[6], (int32_t)q[7]);
                    if (j < m8) store(orow, j, w);
                }
            } else {
#pragma unroll
                for (int i = 0; i < NV; ++i) {
                    const int j = lane + i * 64;
                    if (j < m8) {
                        int32_t q[8];
#pragma unroll
                        for (int e = 0; e < 8; ++e) q[e] = quant_i8_rcp((float)cur[i][e], s, y);
                        uint2_t w;
                        w.x = pack4_i8(q[0], q[1], q[2], q[3]);
                        w.y = pack4_i8(q[4], q[5], q[6], q[7]);
                        store(orow, j, w);
                    }
                }
            }
        }
        if (next >= rows) break;
        load(cur, next);
        row = next;
    }
}

// Workgroups (4 waves each) for k_rows: between 1 and max_k per compute unit (what the register
// budget lets be resident at once), the count that wastes the fewest wave-rows; more workgroups
// on a tie.
static unsigned rows_grid(int64_t rows, int cus, int nv) {
    const int max_k = nv <= 8 ? 8 : 4;
    const int64_t need = ceil_div(rows, 4);
    if (need <= (int64_t)cus) return (unsigned)need;
    int64_t best = cus;

    double best_eff = 0.0;
    for (int k = 1; k <= max_k; ++k) {
        const int64_t g = (int64_t)cus * k;
        if (g > need) break;
        const int64_t per = ceil_div(rows, g * 4);
        const double eff = (double)rows / (double)(per * g * 4);
        if (eff >= best_eff) { best_eff = eff; best = g; }
    }
    return (unsigned)best;
}

template <bool QUANT, bool UA = false>
static void launch_rows(const RowsArgs& ra, int nv, hipStream_t st) {
    const dim3 g(rows_grid(ra.rows0 + ra.rows1, compute_units(), nv));
    if (nv <= 1) hipLaunchKernelGGL((k_rows<1, QUANT, UA>), g, dim3(256), 0, st, ra);
    else if (nv <= 2) hipLaunchKernelGGL((k_rows<2, QUANT, UA>), g, dim3(256), 0, st, ra);
    else if (nv <= 4) hipLaunchKernelGGL((k_rows<4, QUANT, UA>), g, dim3(256), 0, st, ra);
    else if (nv <= 8) hipLaunchKernelGGL((k_rows<8, QUANT, UA>), g, dim3(256), 0, st, ra);
    else hipLaunchKernelGGL((k_rows<16, QUANT, UA>), g, dim3(256), 0, st, ra);
}

static int check3(int32_t batch, int32_t n, int32_t m) {
    if (batch < 0 || n < 0 || m < 0) return CPMK_EBADARG;
    return 0;
}

static int row_absmax(int64_t rows, int32_t m, const void* mat, void* out, hipStream_t st) {
    if (rows == 0) return 0;
    if (out == nullptr || (m > 0 && mat == nullptr)) return CPMK_EBADARG;       // (rows of no elements have no buffer)
    const bool vec = (m % 8 == 0) && aligned16(mat);
    const half_t* p = (const half_t*)mat;
    half_t* o = (half_t*)out;
    // few long rows: a whole block per row; otherwise a wave per row
    const bool wide = rows < 2048 && m >= 2048;
    if (wide) {
        if (vec) hipLaunchKernelGGL((k_row_absmax<256, true>), dim3((unsigned)rows), dim3(256), 0, st, rows, m, p, o);
        else hipLaunchKernelGGL((k_row_absmax<256, false>), dim3((unsigned)rows), dim3(256), 0, st, rows, m, p, o);
    } else {
        const int nv = (int)ceil_div(m, 512);
        if (nv <= 16) {
            const RowsArgs ra = {p, o, nullptr, rows, nullptr, nullptr, nullptr, 0, m};
            if (vec) launch_rows<false>(ra, nv, st);
            else launch_rows<false, true>(ra, nv, st);
            return launch_status();
        }
        if (!grid_fits(ceil_div(rows, 4))) return CPMK_ETOOBIG;
        const unsigned g = (unsigned)ceil_div(rows, 4);
        if (vec) hipLaunchKernelGGL((k_row_absmax<64, true>), dim3(g), dim3(256), 0, st, rows, m, p, o);
        else hipLaunchKernelGGL((k_row_absmax<64, false>), dim3(g), dim3(256), 0, st, rows, m, p, o);
    }
    return launch_status();
}

template <int MODE>
static int round_launch(int32_t batch, int32_t n, int32_t m, const void* mat, const void* scale,
                        void* out, hipStream_t st) {
    const int64_t total = (int64_t)batch * n * m;
    if (total == 0) return 0;
    if (any_null(mat, scale, out)) return CPMK_EBADARG;
    auto low = [](const void* q, uintptr_t mask) { return (reinterpret_cast<uintptr_t>(q) & mask) == 0; };
    const bool vec = (m % 16 == 0) && aligned16(mat) && aligned16(out) && (MODE == 0 || aligned16(scale));
    const bool quads = (m % 4 == 0) && low(mat, 7) && low(out, 3) && (MODE == 0 || low(scale, 7));
    const half_t* p = (const half_t*)mat;
    const half_t* s = (const half_t*)scale;
    int8_t* o = (int8_t*)out;
    if (vec) {
        const int64_t g = ceil_div(total / 16, 256);
        hipLaunchKernelGGL((k_round<MODE, 16>), dim3((unsigned)g), dim3(256), 0, st, total, n, m, p, s, o);
    } else if (quads) {
        const int64_t g = ceil_div(total / 4, 256);
        hipLaunchKernelGGL((k_round<MODE, 4>), dim3((unsigned)g), dim3(256), 0, st, total, n, m, p, s, o);
    } else {
        const int64_t g = ceil_div(total, 256);
        hipLaunchKernelGGL((k_round<MODE, 1>), dim3((unsigned)g), dim3(256), 0, st, total, n, m, p, s, o);
    }
    return launch_status();
}

template <int MODE>
static int dequant_launch(int32_t batch, int32_t n, int32_t m, const void* mat, const void* sx,
                          const void* sy, void* out, int bcx, int bcy, hipStream_t st) {
    const int64_t total = (int64_t)batch * n * m;
    if (total == 0) return 0;
    if (any_null(mat, out) || (MODE != 2 && sx == nullptr) || (MODE != 1 && sy == nullptr)) return CPMK_EBADARG;
    auto low = [](const void* q, uintptr_t mask) { return (reinterpret_cast<uintptr_t>(q) & mask) == 0; };
    const bool vec = (m % 8 == 0) && aligned16(mat) && aligned16(out) && (MODE == 1 || aligned16(sy));
    const bool quads = (m % 4 == 0) && aligned16(mat) && low(out, 7) && (MODE == 1 || low(sy, 7));
    auto go = [&](auto kern, int w) {
        hipLaunchKernelGGL(kern, dim3((unsigned)ceil_div(total / w, 256)), dim3(256), 0, st, total, n, m, (const int32_t*)mat,
                           (const half_t*)sx, (const half_t*)sy, (half_t*)out, bcx, bcy);
    };
    if (vec) go(k_dequant<MODE, 8>, 8);
    else if (quads) go(k_dequant<MODE, 4>, 4);
    else go(k_dequant<MODE, 1>, 1);
    return launch_status();
}

}  // namespace cpmk

using namespace cpmk;

extern "C" {

int cpmk_gemm_quantize_cols(int32_t, int32_t, int32_t, const void*, void*, void*, int, void*);   // colquant.hip

int cpmk_gemm_calc_scale(int32_t batch, int32_t n, int32_t m, const void* mat, void* out, void* stream) {
    clear_stale_error();
    if (int e = check3(batch, n, m)) return e;
    return row_absmax((int64_t)batch * n, m, mat, out, (hipStream_t)stream);
}

int cpmk_gemv_calc_scale(int32_t batch, int32_t n, const void* vec, void* out, void* stream) {
    clear_stale_error();
    if (batch < 0 || n < 0) return CPMK_EBADARG;
    return row_absmax(batch, n, vec, out, (hipStream_t)stream);
}

int cpmk_gemm_calc_scale_transpose(int32_t batch, int32_t n, int32_t m, const void* mat, void* out,
                                   void* stream) {
    clear_stale_error();
    if (int e = check3(batch, n, m)) return e;
    if (batch == 0 || m == 0) return 0;
    if (any_null(out) || (n > 0 && mat == nullptr)) return CPMK_EBADARG;
    if (n > 0) {        // columns in registers, tall ones shared by a team of workgroups
        const int rc = col_absmax_team(batch, n, m, mat, out, stream);
        if (rc >= 0) return rc;
    }
    const bool vec = (m % 8 == 0) && aligned16(mat);
    for (int64_t b0 = 0; b0 < batch; b0 += 65535) {       // (grid y: at most 65535 batch entries per launch)
        const int64_t nb = batch - b0 < 65535 ? batch - b0 : 65535;
        dim3 grid((unsigned)ceil_div(m, 64), (unsigned)nb);
        const half_t* src = (const half_t*)mat + b0 * n * m;
        half_t* dst = (half_t*)out + b0 * m;
        if (vec) hipLaunchKernelGGL((k_col_absmax<true>), grid, dim3(256), 0, (hipStream_t)stream, n, m, src, dst);
        else hipLaunchKernelGGL((k_col_absmax<false>), grid, dim3(256), 0, (hipStream_t)stream, n, m, src, dst);
        if (int e = launch_status()) return e;
    }
    return 0;
}

int cpmk_gemm_round(int32_t batch, int32_t n, int32_t m, const void* mat, const void* scale, void* out,
                    void* stream) {
    clear_stale_error();
    if (int e = check3(batch, n, m)) return e;
    return round_launch<0>(batch, n, m, mat, scale, out, (hipStream_t)stream);
}

int cpmk_gemv_round(int32_t batch, int32_t n, const void* vec, const void* scale, void* out, void* stream) {
    clear_stale_error();
    if (batch < 0 || n < 0) return CPMK_EBADARG;
    return round_launch<0>(1, batch, n, vec, scale, out, (hipStream_t)stream);
}

int cpmk_gemm_round_transpose(int32_t batch, int32_t n, int32_t m, const void* mat, const void* scale,
                              void* out, void* stream) {
    clear_stale_error();
    if (int e = check3(batch, n, m)) return e;
    return round_launch<1>(batch, n, m, mat, scale, out, (hipStream_t)stream);
}

int cpmk_gemm_scale(int32_t batch, int32_t n, int32_t m, const void* mat, const void* scale_x,
                    const void* scale_y, void* out, int bcx, int bcy, void* stream) {
    clear_stale_error();
    if (int e = check3(batch, n, m)) return e;
    return dequant_launch<0>(batch, n, m, mat, scale_x, scale_y, out, bcx, bcy, (hipStream_t)stream);
}

int cpmk_gemm_scale_x(int32_t batch, int32_t n, int32_t m, const void* mat, const void* scale_x, void* out,
                      void* stream) {
    clear_stale_error();
    if (int e = check3(batch, n, m)) return e;
    return dequant_launch<1>(batch, n, m, mat, scale_x, nullptr, out, 0, 0, (hipStream_t)stream);
}

int cpmk_gemm_scale_y(int32_t batch, int32_t n, int32_t m, const void* mat, const void* scale_y, void* out,
                      void* stream) {
    clear_stale_error();
    if (int e = check3(batch, n, m)) return e;
    return dequant_launch<2>(batch, n, m, mat, nullptr, scale_y, out, 0, 0, (hipStream_t)stream);
}

int cpmk_gemm_quantize(int32_t batch, int32_t n, int32_t m, const void* mat, void* scale, void* out,
                       int transpose, void* stream) {
    clear_stale_error();
    if (int e = check3(batch, n, m)) return e;
    hipStream_t st = (hipStream_t)stream;
    if (!transpose) {
        const int64_t rows = (int64_t)batch * n;
        if (rows == 0) return 0;
        if (any_null(scale) || (m > 0 && any_null(mat, out))) return CPMK_EBADARG;
        const bool vec = (m % 8 == 0) && aligned16(mat) && ((reinterpret_cast<uintptr_t>(out) & 7u) == 0);
        if (m > 0 && m <= 64 * 8 * 16) {
            const RowsArgs ra = {(const half_t*)mat, (half_t*)scale, (int8_t*)out, rows, nullptr, nullptr, nullptr, 0, m};
            if (vec) launch_rows<true>(ra, (int)ceil_div(m, 512), st);
            else launch_rows<true, true>(ra, (int)ceil_div(m, 512), st);
            return launch_status();
        }
        if (int e = cpmk_gemm_calc_scale(batch, n, m, mat, scale, stream)) return e;
        return cpmk_gemm_round(batch, n, m, mat, scale, out, stream);
    }
    return cpmk_gemm_quantize_cols(batch, n, m, mat, scale, out, 0, stream);
}

int cpmk_gemm_quantize_pair(int64_t rows0, const void* mat0, void* scale0, void* out0, int64_t rows1, const void* mat1,
                            void* scale1, void* out1, int32_t m, void* stream) {
    clear_stale_error();
    if (rows0 < 0 || rows1 < 0 || m < 0 || rows0 > 0x7fffffff || rows1 > 0x7fffffff) return CPMK_EBADARG;
    if (m == 0 || rows0 + rows1 == 0) return 0;
    if ((rows0 > 0 && any_null(mat0, scale0, out0)) || (rows1 > 0 && any_null(mat1, scale1, out1))) return CPMK_EBADARG;
    const bool vec = (m % 8 == 0) && (rows0 == 0 || (aligned16(mat0) && (reinterpret_cast<uintptr_t>(out0) & 7u) == 0)) &&
                     (rows1 == 0 || (aligned16(mat1) && (reinterpret_cast<uintptr_t>(out1) & 7u) == 0));
    if (m <= 64 * 8 * 16) {
        const RowsArgs ra = {(const half_t*)mat0, (half_t*)scale0, (int8_t*)out0, rows0,
                             (const half_t*)mat1, (half_t*)scale1, (int8_t*)out1, rows1, m};
        if (vec) launch_rows<true>(ra, (int)ceil_div(m, 512), (hipStream_t)stream);
        else launch_rows<true, true>(ra, (int)ceil_div(m, 512), (hipStream_t)stream);
        return launch_status();
    }
    if (rows0 > 0)
        if (int e = cpmk_gemm_quantize(1, (int32_t)rows0, m, mat0, scale0, out0, 0, stream)) return e;
    if (rows1 > 0) return cpmk_gemm_quantize(1, (int32_t)rows1, m, mat1, scale1, out1, 0, stream);
    return 0;
}

}  // extern "C"
