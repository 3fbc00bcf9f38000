// Register-resident column tiles for reductions over dim 1 of a (batch, n, m) fp16 tensor.
//
// The reference walks such tensors with 32x32 thread blocks, 64-byte row segments and two or
// three passes over global memory (cuda/layernorm.cu:6-71, cuda/softmax.cu:6-43).  Here one
// workgroup of NT threads owns all n rows of LPR*8 adjacent columns and keeps them in
// registers, so HBM is read once and written once:
//   lane -> (cg = tid % LPR, rg = tid / LPR); pass p covers rows p*(NT/LPR) + rg;
//   each lane holds R 16-byte pieces (8 columns of R rows).
// Reductions run per lane, then over the lanes of a wave that share cg (xor butterflies on
// the lane bits above log2(LPR)), then over waves through a few hundred bytes of LDS.
#pragma once
#include "common.h"

namespace cpmk {

template <int NT, int LPR, int R>
struct ColTile {
    static constexpr int RPP = NT / LPR;       // rows per pass
    static constexpr int ROWS = RPP * R;       // rows the tile can hold
    static constexpr int COLS = LPR * 8;
    static constexpr int NW = NT / 64;
    // LDS floats needed by reduce<NV>: (NW + 1) * COLS * NV
};

// Load the tile; rows >= n and columns >= m are left as `fill` in every half.  `base` is the
// (wave-uniform) start of this batch entry; element offsets inside it are 32-bit, which lets
// the compiler address with a scalar base plus one VGPR offset instead of holding R 64-bit
// pointers across the reduction phases (callers guarantee n*m < 2^31).
//
// NTL / NTS: non-temporal loads / stores.  Only for tiles whose row segments are whole 128-byte cache
// lines (LPR == 8) and for data that is not read again soon: a segment shorter than a line is completed
// by a neighbouring workgroup, so it has to allocate in L2.
//
// UA: rows that are not whole 16-byte pieces, or buffers that are not 16-byte aligned.  A piece inside its row still
// moves as one 16-byte access (global accesses need no alignment; one that crosses a cache line costs a second
// request), the piece across a row's end in at most three narrower ones.
template <int NT, int LPR, int R, bool NTL = false, bool UA = false>
__device__ inline void coltile_load(half8_t (&v)[R], const half_t* base, int32_t n, int32_t m, int32_t col0,
                                    half_t fill) {
    constexpr int RPP = NT / LPR;
    const int rg = threadIdx.x / LPR;
    const uint32_t off0 = (uint32_t)rg * (uint32_t)m + (uint32_t)col0, stride = (uint32_t)RPP * (uint32_t)m;
    if constexpr (UA) {
        if (col0 + 8 <= m) {        // the lane's pieces lie inside their rows
#pragma unroll
            for (int p = 0; p < R; ++p) {
                half8_t x;
#pragma unroll
                for (int e = 0; e < 8; ++e) x[e] = fill;
                if (p * RPP + rg < n) x = load_half8_any(base + (off0 + p * stride));
                v[p] = x;
            }
        } else {                    // ... or across their ends (the first m % 8 columns of the piece), or past them
            const bool tail = col0 < m;
#pragma unroll
            for (int p = 0; p < R; ++p) {
                half8_t x;
#pragma unroll
                for (int e = 0; e < 8; ++e) x[e] = fill;
                if (tail && p * RPP + rg < n) x = load_half8_head_any(base + (off0 + p * stride), m & 7, x);
                v[p] = x;
            }
        }
    } else {
#pragma unroll
        for (int p = 0; p < R; ++p) {
            const int32_t row = p * RPP + rg;
            half8_t x;
#pragma unroll
            for (int e = 0; e < 8; ++e) x[e] = fill;
            if (row < n && col0 < m) {
                const half8_t* src = reinterpret_cast<const half8_t*>(base + (off0 + p * stride));
                x = NTL ? __builtin_nontemporal_load(src) : *src;
            }
            v[p] = x;
        }
    }
}

template <int NT, int LPR, int R, bool NTS = false, bool UA = false>
__device__ inline void coltile_store(const half8_t (&v)[R], half_t* base, int32_t n, int32_t m, int32_t col0) {
    constexpr int RPP = NT / LPR;
    const int rg = threadIdx.x / LPR;
    const uint32_t off0 = (uint32_t)rg * (uint32_t)m + (uint32_t)col0, stride = (uint32_t)RPP * (uint32_t)m;
    if constexpr (UA) {
        if (col0 + 8 <= m) {
#pragma unroll
            for (int p = 0; p < R; ++p)
                if (p * RPP + rg < n) store_half8_any(base + (off0 + p * stride), v[p]);
        } else if (col0 < m) {
#pragma unroll
            for (int p = 0; p < R; ++p)
                if (p * RPP + rg < n) store_half8_head_any(base + (off0 + p * stride), m & 7, v[p]);
        }
    } else {
#pragma unroll
        for (int p = 0; p < R; ++p) {
            const int32_t row = p * RPP + rg;
            if (row < n && col0 < m) {
                half8_t* dst = reinterpret_cast<half8_t*>(base + (off0 + p * stride));
                if (NTS) __builtin_nontemporal_store(v[p], dst);
                else *dst = v[p];
            }
        }
    }
}

// v combined (sum or maximum) over the eight lanes of a wave that share lane % 8 -- lanes l, l ^ 8, l ^ 16, l ^ 32
// in that order, as three rounds of __shfl_xor would -- without the trips through the LDS crossbar: a rotation by
// 8 within each row of 16 lanes as an operand modifier, then the two lane-swap instructions of this architecture
// (v_permlane16_swap: odd rows of one register against even rows of the other; v_permlane32_swap: the halves).
template <bool IS_MAX>
__device__ __forceinline__ float lanes_mod8_combine(float v) {
    auto op = [](float a, float b) __attribute__((always_inline)) { return IS_MAX ? fmaxf(a, b) : a + b; };
    const uint32_t b0 = __builtin_bit_cast(uint32_t, v);
    v = op(v, __builtin_bit_cast(float, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)b0, 0x128, 0xf, 0xf, true)));      // row_ror:8
    const uint32_t b1 = __builtin_bit_cast(uint32_t, v);
    const auto r = __builtin_amdgcn_permlane16_swap(b1, b1, false, false);
    v = op(__builtin_bit_cast(float, (uint32_t)r[0]), __builtin_bit_cast(float, (uint32_t)r[1]));
    const uint32_t b2 = __builtin_bit_cast(uint32_t, v);
    const auto q = __builtin_amdgcn_permlane32_swap(b2, b2, false, false);
    return op(__builtin_bit_cast(float, (uint32_t)q[0]), __builtin_bit_cast(float, (uint32_t)q[1]));
}

// Reduce NV groups of 8 per-lane column partials over all rows of the tile.  On return every
// lane holds the totals of its own 8 columns.  `lds` must hold (NT/64 + 1) * LPR*8 * NV floats.
template <int NT, int LPR, int NV, bool IS_MAX>
__device__ inline void coltile_reduce(float (&v)[NV * 8], float* lds) {
    constexpr int NW = NT / 64, COLS = LPR * 8, W = COLS * NV;
    if constexpr (LPR == 8 && !IS_MAX) {        // (for the maxima of the column quantiser the lane-swap form measured 4 % slower than the shuffles)
#pragma unroll
        for (int e = 0; e < NV * 8; ++e) v[e] = lanes_mod8_combine<IS_MAX>(v[e]);
    } else {
#pragma unroll
        for (int o = LPR; o < 64; o <<= 1) {
#pragma unroll
            for (int e = 0; e < NV * 8; ++e) {
                const float t = __shfl_xor(v[e], o, kWave);
                v[e] = IS_MAX ? fmaxf(v[e], t) : v[e] + t;
            }
        }
    }
    if (NW == 1) return;
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    if (lane < LPR) {
#pragma unroll
        for (int g = 0; g < NV; ++g)
#pragma unroll
            for (int e = 0; e < 8; ++e) lds[w * W + g * COLS + lane * 8 + e] = v[g * 8 + e];
    }
    __syncthreads();
    if (tid < W) {
        float r = lds[tid];
#pragma unroll
        for (int i = 1; i < NW; ++i) r = IS_MAX ? fmaxf(r, lds[i * W + tid]) : r + lds[i * W + tid];
        lds[NW * W + tid] = r;
    }
    __syncthreads();
    const int cg = tid % LPR;
#pragma unroll
    for (int g = 0; g < NV; ++g)
#pragma unroll
        for (int e = 0; e < 8; ++e) v[g * 8 + e] = lds[NW * W + g * COLS + cg * 8 + e];
    __syncthreads();
}

// The same reduction for kernels that only hand the totals on (to their team): thread i < COLS*NV
// calls sink(i, total of packet i) -- packet g*COLS + c is statistic g of tile column c -- and
// nothing is read back, which saves two barriers.  Needs more than one wave.
template <int NT, int LPR, int NV, bool IS_MAX, class F>
__device__ inline void coltile_reduce_to(float (&v)[NV * 8], float* lds, F&& sink) {
    constexpr int NW = NT / 64, COLS = LPR * 8, W = COLS * NV;
    static_assert(NW > 1, "one wave has nothing to combine");
    if constexpr (LPR == 8 && !IS_MAX) {        // (for the maxima of the column quantiser the lane-swap form measured 4 % slower than the shuffles)
#pragma unroll
        for (int e = 0; e < NV * 8; ++e) v[e] = lanes_mod8_combine<IS_MAX>(v[e]);
    } else {
#pragma unroll
        for (int o = LPR; o < 64; o <<= 1) {
#pragma unroll
            for (int e = 0; e < NV * 8; ++e) {
                const float t = __shfl_xor(v[e], o, kWave);
                v[e] = IS_MAX ? fmaxf(v[e], t) : v[e] + t;
            }
        }
    }
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    if (lane < LPR) {
#pragma unroll
        for (int g = 0; g < NV; ++g)
#pragma unroll
            for (int e = 0; e < 8; ++e) lds[w * W + g * COLS + lane * 8 + e] = v[g * 8 + e];
    }
    __syncthreads();
    if (tid < W) {
        float r = lds[tid];
#pragma unroll
        for (int i = 1; i < NW; ++i) r = IS_MAX ? fmaxf(r, lds[i * W + tid]) : r + lds[i * W + tid];
        sink(tid, r);
    }
}

}  // namespace cpmk
