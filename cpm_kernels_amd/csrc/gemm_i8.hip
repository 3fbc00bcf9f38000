// int8 x int8 -> int32 batched GEMM on the CDNA4 matrix cores, optionally with the fp16
// dequantising epilogue applied to the accumulators in registers.
//
// Replaces the cuBLASLt call of the reference (cpm_kernels/kernels/gemm.py:127-186).  In
// row-major terms that call computes, per batch,
//     out[j, i] = sum_kk  Bop[j, kk] * Aop[i, kk]        j < n, i < m
// with Bop = B (n,k) if !bT else B^T of a (k,n) array, Aop = A^T of a (k,m) array if !aT
// else A (m,k).  Inside this file the operand indexed by the output ROW j is called P and
// the one indexed by the output COLUMN i is called Q; each is either "K-major" (kk
// contiguous) or "MN-major" (j resp. i contiguous).
//
// Fast kernel (k_gemm_kmajor): both operands K-major, k % 16 == 0.  256-thread workgroups,
// 64-byte K slices staged through double-buffered, XOR-swizzled LDS, v_mfma_i32_32x32x32_i8
// with the output row operand as MFMA "A" and the output column operand as MFMA "B" so that
// 32 lanes store 32 consecutive output columns.  Integer accumulation is exact, so any
// summation order gives the reference's int32 result bit for bit.
//
// Generic kernel (k_gemm_generic): any layout, any sizes; LDS tiles + v_dot4_i32_i8.
#include "common.h"

namespace cpmk {

struct GemmArgs {
    const int8_t* P;      // row operand
    const int8_t* Q;      // column operand
    void* out;            // int32 or fp16, (batch, n, m)
    const half_t* srow;   // fused epilogue: scale per output row j
    const half_t* scol;   // fused epilogue: scale per output column i
    int64_t strideP, strideQ;   // batch strides in bytes (0 = broadcast)
    int32_t n, m, k;
    int32_t bc_row, bc_col;
    int32_t tiles_r, tiles_c;
};

// ---------------------------------------------------------------------------------------
// Fast path
// ---------------------------------------------------------------------------------------
constexpr int BK = 64;   // bytes of K per LDS stage

// 16-byte chunk c (0..3) of LDS row r lives at chunk slot c ^ ((r >> 2) & 3): sixteen
// consecutive rows reading the same logical chunk then cover all 64 banks exactly once.
__device__ inline int lds_off(int r, int c) { return r * BK + ((c ^ ((r >> 2) & 3)) << 4); }

template <int WAVES_R, int WAVES_C, int TR, int TC, bool FUSED>
__global__ __launch_bounds__(WAVES_R* WAVES_C * 64) void k_gemm_kmajor(GemmArgs a) {
    constexpr int NT = WAVES_R * WAVES_C * 64;
    constexpr int BR = WAVES_R * TR * 32;   // output rows per workgroup
    constexpr int BC = WAVES_C * TC * 32;   // output columns per workgroup
    constexpr int CH_P = BR * (BK / 16) / NT;   // 16-byte chunks per thread, P tile
    constexpr int CH_Q = BC * (BK / 16) / NT;
    static_assert(BR * (BK / 16) % NT == 0 && BC * (BK / 16) % NT == 0, "tile/threads mismatch");

    extern __shared__ __attribute__((aligned(16))) int8_t smem[];
    constexpr int STAGE = (BR + BC) * BK;   // stage s: P tile at s*STAGE, Q tile after it

    // tile rasterisation: XCD-aware, then column-tile-fastest inside groups of 8 row tiles
    const uint32_t ntiles = (uint32_t)a.tiles_r * a.tiles_c;
    uint32_t t = xcd_remap(blockIdx.x, ntiles);
    constexpr uint32_t GR = 4;   // row tiles per raster group
    const uint32_t group_sz = GR * a.tiles_c;
    const uint32_t g = t / group_sz;
    const uint32_t rows_in_group = min(GR, (uint32_t)a.tiles_r - g * GR);
    const uint32_t tin = t - g * group_sz;
    const uint32_t tile_r = g * GR + tin % rows_in_group;
    const uint32_t tile_c = tin / rows_in_group;
    const int32_t j0 = tile_r * BR, i0 = tile_c * BC;

    const int b = blockIdx.z;
    const int8_t* P = a.P + (int64_t)b * a.strideP;
    const int8_t* Q = a.Q + (int64_t)b * a.strideQ;
    const int32_t K = a.k;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wr = wave / WAVES_C, wc = wave % WAVES_C;

    // global -> register staging: chunk id q = tid + s*NT -> row q/4, chunk q%4
    int4_t gp[CH_P], gq[CH_Q];
    auto gload = [&](int32_t k0) {
#pragma unroll
        for (int s = 0; s < CH_P; ++s) {
            const int q = tid + s * NT, r = q >> 2, c = q & 3;
            const int32_t row = j0 + r, kc = k0 + c * 16;
            int4_t v = {0, 0, 0, 0};
            if (row < a.n && kc < K) v = *reinterpret_cast<const int4_t*>(P + (int64_t)row * K + kc);
            gp[s] = v;
        }
#pragma unroll
        for (int s = 0; s < CH_Q; ++s) {
            const int q = tid + s * NT, r = q >> 2, c = q & 3;
            const int32_t row = i0 + r, kc = k0 + c * 16;
            int4_t v = {0, 0, 0, 0};
            if (row < a.m && kc < K) v = *reinterpret_cast<const int4_t*>(Q + (int64_t)row * K + kc);
            gq[s] = v;
        }
    };
    auto sstore = [&](int buf) {
#pragma unroll
        for (int s = 0; s < CH_P; ++s) {
            const int q = tid + s * NT, r = q >> 2, c = q & 3;
            *reinterpret_cast<int4_t*>(smem + buf * STAGE + lds_off(r, c)) = gp[s];
        }
#pragma unroll
        for (int s = 0; s < CH_Q; ++s) {
            const int q = tid + s * NT, r = q >> 2, c = q & 3;
            *reinterpret_cast<int4_t*>(smem + buf * STAGE + BR * BK + lds_off(r, c)) = gq[s];
        }
    };

    int16_tv acc[TR][TC];
#pragma unroll
    for (int i = 0; i < TR; ++i)
#pragma unroll
        for (int j = 0; j < TC; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

    const int nk = (K + BK - 1) / BK;
    gload(0);
    sstore(0);
    __syncthreads();

    const int lrow = lane & 31, lk = lane >> 5;
    for (int it = 0; it < nk; ++it) {
        const int cur = it & 1;
        if (it + 1 < nk) gload((it + 1) * BK);
#pragma unroll
        for (int ks = 0; ks < BK / 32; ++ks) {
            int4_t fa[TR], fb[TC];
#pragma unroll
            for (int i = 0; i < TR; ++i)
                fa[i] = *reinterpret_cast<const int4_t*>(smem + cur * STAGE + lds_off(wr * TR * 32 + i * 32 + lrow, ks * 2 + lk));
#pragma unroll
            for (int j = 0; j < TC; ++j)
                fb[j] = *reinterpret_cast<const int4_t*>(smem + cur * STAGE + BR * BK + lds_off(wc * TC * 32 + j * 32 + lrow, ks * 2 + lk));
#pragma unroll
            for (int i = 0; i < TR; ++i)
#pragma unroll
                for (int j = 0; j < TC; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        if (it + 1 < nk) sstore(cur ^ 1);
        __syncthreads();
    }

    // epilogue: accumulator register e of lane l is output row (e/4)*8 + (l/32)*4 + e%4,
    // column l%32 of its 32x32 tile.
    const int64_t obase = (int64_t)b * a.n * a.m;
#pragma unroll
    for (int i = 0; i < TR; ++i) {
#pragma unroll
        for (int j = 0; j < TC; ++j) {
            const int32_t col = i0 + wc * TC * 32 + j * 32 + lrow;
            float sy = 0.0f;
            if (FUSED && col < a.m) sy = (float)a.scol[(a.bc_col ? 0 : (int64_t)b * a.m) + col];
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int32_t row = j0 + wr * TR * 32 + i * 32 + (e >> 2) * 8 + lk * 4 + (e & 3);
                if (row < a.n && col < a.m) {
                    const int64_t o = obase + (int64_t)row * a.m + col;
                    if (FUSED) {
                        const float sx = (float)a.srow[a.bc_row ? row : (int64_t)b * a.n + row];
                        reinterpret_cast<half_t*>(a.out)[o] = dequant(acc[i][j][e], sx, sy);
                    } else {
                        reinterpret_cast<int32_t*>(a.out)[o] = acc[i][j][e];
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------
// Generic path: 64x64 output tile, 32 bytes of K per stage, 256 threads each computing a
// 4x4 block with v_dot4_i32_i8.  Element-wise guarded loads handle every layout and size.
// ---------------------------------------------------------------------------------------
template <bool FUSED>
__global__ __launch_bounds__(256) void k_gemm_generic(GemmArgs a, int p_kmajor, int q_kmajor) {
    constexpr int T = 64, GK = 32, LD = GK + 4;
    __shared__ __attribute__((aligned(4))) int8_t sP[T * LD];
    __shared__ __attribute__((aligned(4))) int8_t sQ[T * LD];
    const int b = blockIdx.z;
    const int8_t* P = a.P + (int64_t)b * a.strideP;
    const int8_t* Q = a.Q + (int64_t)b * a.strideQ;
    const int32_t j0 = blockIdx.y * T, i0 = blockIdx.x * T;
    const int tid = threadIdx.x, ty = tid >> 4, tx = tid & 15;
    int32_t acc[4][4];
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[r][c] = 0;

    for (int32_t k0 = 0; k0 < a.k; k0 += GK) {
#pragma unroll
        for (int s = 0; s < T * GK / 256; ++s) {
            const int q = tid + s * 256;
            int r, kk;
            if (p_kmajor) { r = q / GK; kk = q % GK; } else { r = q % T; kk = q / T; }
            const int32_t row = j0 + r, kg = k0 + kk;
            int8_t v = 0;
            if (row < a.n && kg < a.k) v = p_kmajor ? P[(int64_t)row * a.k + kg] : P[(int64_t)kg * a.n + row];
            sP[r * LD + kk] = v;
            if (q_kmajor) { r = q / GK; kk = q % GK; } else { r = q % T; kk = q / T; }
            const int32_t col = i0 + r, kg2 = k0 + kk;
            v = 0;
            if (col < a.m && kg2 < a.k) v = q_kmajor ? Q[(int64_t)col * a.k + kg2] : Q[(int64_t)kg2 * a.m + col];
            sQ[r * LD + kk] = v;
        }
        __syncthreads();
#pragma unroll
        for (int k4 = 0; k4 < GK / 4; ++k4) {
            int32_t pa[4], qb[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) pa[r] = *reinterpret_cast<const int32_t*>(sP + (ty * 4 + r) * LD + k4 * 4);
#pragma unroll
            for (int c = 0; c < 4; ++c) qb[c] = *reinterpret_cast<const int32_t*>(sQ + (tx + c * 16) * LD + k4 * 4);
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int c = 0; c < 4; ++c) acc[r][c] = __builtin_amdgcn_sdot4(pa[r], qb[c], acc[r][c], false);
        }
        __syncthreads();
    }
    const int64_t obase = (int64_t)b * a.n * a.m;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int32_t row = j0 + ty * 4 + r;
        if (row >= a.n) continue;
        float sx = 0.0f;
        if (FUSED) sx = (float)a.srow[a.bc_row ? row : (int64_t)b * a.n + row];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int32_t col = i0 + tx + c * 16;
            if (col >= a.m) continue;
            const int64_t o = obase + (int64_t)row * a.m + col;
            if (FUSED) {
                const float sy = (float)a.scol[(a.bc_col ? 0 : (int64_t)b * a.m) + col];
                reinterpret_cast<half_t*>(a.out)[o] = dequant(acc[r][c], sx, sy);
            } else {
                reinterpret_cast<int32_t*>(a.out)[o] = acc[r][c];
            }
        }
    }
}

template <int WAVES_R, int WAVES_C, int TR, int TC, bool FUSED>
static int launch_kmajor(GemmArgs& a, int batch, hipStream_t st) {
    constexpr int BR = WAVES_R * TR * 32, BC = WAVES_C * TC * 32;
    constexpr int smem = 2 * (BR + BC) * BK;
    a.tiles_r = (int32_t)ceil_div(a.n, BR);
    a.tiles_c = (int32_t)ceil_div(a.m, BC);
    auto kern = k_gemm_kmajor<WAVES_R, WAVES_C, TR, TC, FUSED>;
    static bool attr_set = false;   // raising the dynamic LDS limit is idempotent
    if (!attr_set && smem > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, smem);
        if (e != hipSuccess) return (int)e;
        attr_set = true;
    }
    dim3 grid((unsigned)(a.tiles_r * a.tiles_c), 1, (unsigned)batch);
    hipLaunchKernelGGL(kern, grid, dim3(WAVES_R * WAVES_C * 64), smem, st, a);
    return launch_status();
}

template <bool FUSED>
static int gemm_dispatch(int32_t m, int32_t k, int32_t n, int32_t batchA, int32_t batchB, int aT, int bT,
                         const void* A, const void* B, const void* srow, const void* scol, int bcr,
                         int bcc, void* out, hipStream_t st) {
    if (m < 0 || n < 0 || k < 0 || batchA < 1 || batchB < 1) return CPMK_EBADARG;
    if ((m % 4) || (n % 4) || (k % 4)) return CPMK_EALIGN;      // kernels/gemm.py:139
    if (!(batchA == batchB || batchA == 1 || batchB == 1)) return CPMK_EBADARG;   // :140
    const int batch = batchA > batchB ? batchA : batchB;
    if (m == 0 || n == 0) return 0;
    if (batch > 65535) return CPMK_ETOOBIG;
    GemmArgs a;
    a.P = (const int8_t*)B; a.Q = (const int8_t*)A; a.out = out;
    a.srow = (const half_t*)srow; a.scol = (const half_t*)scol;
    a.strideP = batchB == 1 ? 0 : (int64_t)n * k;
    a.strideQ = batchA == 1 ? 0 : (int64_t)m * k;
    a.n = n; a.m = m; a.k = k; a.bc_row = bcr; a.bc_col = bcc;
    a.tiles_r = a.tiles_c = 0;
    const bool p_kmajor = !bT, q_kmajor = aT != 0;
    const bool fast = p_kmajor && q_kmajor && k > 0 && (k % 16 == 0) && aligned16(A) && aligned16(B);
    if (fast) {
        // tile choice: large tiles when they still give every CU work, else smaller ones
        const int64_t t256 = ceil_div(n, 256) * ceil_div(m, 128) * batch;
        if (t256 >= 256) return launch_kmajor<2, 2, 4, 2, FUSED>(a, batch, st);
        return launch_kmajor<2, 2, 2, 2, FUSED>(a, batch, st);
    }
    dim3 grid((unsigned)ceil_div(m, 64), (unsigned)ceil_div(n, 64), (unsigned)batch);
    if (grid.y > 65535) return CPMK_ETOOBIG;
    hipLaunchKernelGGL((k_gemm_generic<FUSED>), grid, dim3(256), 0, st, a, (int)p_kmajor, (int)q_kmajor);
    return launch_status();
}

}  // namespace cpmk

using namespace cpmk;

extern "C" {

int cpmk_gemm_int8(int32_t m, int32_t k, int32_t n, int32_t batchA, int32_t batchB, int aT, int bT,
                   const void* A, const void* B, void* out, void* stream) {
    clear_stale_error();
    return gemm_dispatch<false>(m, k, n, batchA, batchB, aT, bT, A, B, nullptr, nullptr, 0, 0, out,
                                (hipStream_t)stream);
}

int cpmk_gemm_int8_scale(int32_t m, int32_t k, int32_t n, int32_t batchA, int32_t batchB, int aT, int bT,
                         const void* A, const void* B, const void* scale_row, const void* scale_col,
                         int broad_cast_row, int broad_cast_col, void* out, void* stream) {
    clear_stale_error();
    return gemm_dispatch<true>(m, k, n, batchA, batchB, aT, bT, A, B, scale_row, scale_col, broad_cast_row,
                               broad_cast_col, out, (hipStream_t)stream);
}

}  // extern "C"
