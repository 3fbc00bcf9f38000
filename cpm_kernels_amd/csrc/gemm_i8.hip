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
// Three kernels, all exact (integer accumulation is order-independent, so the int32 result
// equals the reference's bit for bit):
//   k_gemm_dma     both operands K-major, k % 128 == 0: persistent workgroups walk the output
//                  tiles; global memory goes straight into a ring of XOR-swizzled LDS stages
//                  (global_load_lds_dwordx4), one barrier per 128-byte K slab, fragments read
//                  ahead of their MFMAs, v_mfma_i32_16x16x64_i8 (256x256 tiles) or
//                  v_mfma_i32_32x32x32_i8 (smaller tiles) with the operands swapped so that a lane
//                  owns 4 consecutive output columns; results leave through a per-wave LDS strip
//                  as whole 128-byte lines.
//                  With template parameter LAY it also takes operands stored with K as the row index
//                  (rows of whole 16-byte pieces), gathering the MFMA fragments element by element.
//   k_gemm_kmajor  both operands K-major, k % 16 == 0 (16-byte loads) or any k % 4 == 0 (4-byte loads): register-staged 64-byte K slabs.
//   k_gemm_generic any layout and size: LDS tiles + v_dot4_i32_i8.
// The tile kernel also serves the fp16 product of kernels/gemm.py:188-256 (cpmk_gemm_fp16): the
// same bytes of K per lane feed v_mfma_f32_16x16x32_f16 / v_mfma_f32_32x32x16_f16, with fp32 accumulators.
#include "common.h"
#include <type_traits>

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
    int32_t edge_in;      // bit 0 / 1: the last row / column tile starts at n - BR / m - BC instead of reaching past the end
};

// ---------------------------------------------------------------------------------------
// Fast path
// ---------------------------------------------------------------------------------------
constexpr int BK = 64;   // bytes of K per LDS stage

// 16-byte chunk c (0..3) of LDS row r lives at chunk slot c ^ ((r >> 2) & 3): sixteen
// consecutive rows reading the same logical chunk then cover all 64 banks exactly once.
__device__ inline int lds_off(int r, int c) { return r * BK + ((c ^ ((r >> 2) & 3)) << 4); }

// DW: rows that are only 4-byte aligned (k % 16 != 0): a whole 16-byte piece still comes in one load (global loads of
// four dwords need dword alignment only), the piece across the end of K as single dwords, zero past the end.
struct __attribute__((aligned(4))) Int4Dword { int32_t x, y, z, w; };

template <int WAVES_R, int WAVES_C, int TR, int TC, bool FUSED, bool DW = false>
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
    auto piece = [&](const int8_t* rowp, int32_t kc) __attribute__((always_inline)) {      // bytes [kc, kc + 16) of a row, zeros past K
        int4_t v = {0, 0, 0, 0};
        if constexpr (DW) {
            if (kc + 16 <= K) {
                const Int4Dword t = *reinterpret_cast<const Int4Dword*>(rowp + kc);
                v = int4_t{t.x, t.y, t.z, t.w};
            } else {
#pragma unroll
                for (int d = 0; d < 3; ++d)
                    if (kc + 4 * d < K) v[d] = *reinterpret_cast<const int32_t*>(rowp + kc + 4 * d);
            }
        } else {
            if (kc < K) v = *reinterpret_cast<const int4_t*>(rowp + kc);
        }
        return v;
    };
    auto gload = [&](int32_t k0) {
#pragma unroll
        for (int s = 0; s < CH_P; ++s) {
            const int q = tid + s * NT, r = q >> 2, c = q & 3;
            const int32_t row = j0 + r;
            gp[s] = row < a.n ? piece(P + (int64_t)row * K, k0 + c * 16) : int4_t{0, 0, 0, 0};
        }
#pragma unroll
        for (int s = 0; s < CH_Q; ++s) {
            const int q = tid + s * NT, r = q >> 2, c = q & 3;
            const int32_t row = i0 + r;
            gq[s] = row < a.m ? piece(Q + (int64_t)row * K, k0 + c * 16) : int4_t{0, 0, 0, 0};
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
// Persistent LDS-DMA kernel
// ---------------------------------------------------------------------------------------
template <int X, int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (X < N) {
        f(std::integral_constant<int, X>{});
        static_for<X + 1, N>(f);
    }
}

// What the tile kernel does with its accumulators.
constexpr int kEpiInt32 = 0;     // int8 product, int32 out
constexpr int kEpiDequant = 1;   // int8 product, fp16( (f32(acc) * s_row) * s_col ) out
constexpr int kEpiF16 = 2;       // fp16 product with fp32 accumulation, fp16 out

struct DmaArgs {
    GemmArgs g;
    int32_t batch;
    int32_t ntiles;    // full-size tiles per batch entry (tiles_r x tiles_c)
    uint32_t nfull;    // work items [0, nfull) are whole tiles in walk order ...
    uint32_t nhalf;    // ... items [nfull, nfull + nhalf) are row halves (top, bottom) of the tiles that follow
};

// One work item of the persistent kernel: a whole BR x BC tile, or its top/bottom half.
struct GemmItem {
    uint32_t b;        // batch entry
    int32_t j0, i0;    // first output row / column
    bool half;
    bool valid;
};

// Tiles are walked in groups of GRP row tiles, column-major inside a group, so neighbours in the
// walk share operand slabs in L2.
template <int BR, int BC>
__device__ __forceinline__ GemmItem gemm_item(uint32_t L, const DmaArgs& da) {
    GemmItem it;
    it.valid = L < da.nfull + da.nhalf;
    it.half = L >= da.nfull;
    const uint32_t h = it.half ? L - da.nfull : 0;
    const uint32_t id = it.half ? da.nfull + (h >> 1) : L;
    it.b = id / (uint32_t)da.ntiles;
    const uint32_t t = id - it.b * (uint32_t)da.ntiles;
    constexpr uint32_t GRP = 4;
    const uint32_t group_sz = GRP * (uint32_t)da.g.tiles_c;
    const uint32_t g = t / group_sz;
    const uint32_t rows_in_group = min(GRP, (uint32_t)da.g.tiles_r - g * GRP);
    const uint32_t tin = t - g * group_sz;
    it.j0 = (int32_t)((g * GRP + tin % rows_in_group) * BR + (h & 1) * (BR / 2));
    it.i0 = (int32_t)((tin / rows_in_group) * BC);
    // An operand stored (K, rows) whose rows are not whole 16-byte pieces cannot be read past the matrix's edge piece by
    // piece: its last tile then lies inside the matrix and overlaps its neighbour, whose outputs it computes again
    // (the same bits, stored twice).
    if (da.g.edge_in & 1) it.j0 = min(it.j0, da.g.n - BR);
    if (da.g.edge_in & 2) it.i0 = min(it.i0, da.g.m - BC);
    return it;
}

// A 16-byte piece of an output row on its way to memory; `left` = elements from the piece's first to the end of
// the row (a multiple of 4, at least 4).  int32 rows and fp16 rows of a multiple of 8 elements keep every piece
// whole and 16-byte aligned.  fp16 rows of 8j + 4 elements are only 8-byte aligned from one row to the next and
// end in half a piece: such pieces leave as 8-byte halves.
template <int ESZ>
__device__ __forceinline__ void store_piece(int8_t* dst, int4_t v, int32_t left) {
    if (ESZ == 4 || ((reinterpret_cast<uintptr_t>(dst) & 15u) == 0 && left >= 8)) {
        *reinterpret_cast<int4_t*>(dst) = v;       // (the non-temporal hint changes nothing here: 133.7 against 134.1-135.2 us)
    } else {
        *reinterpret_cast<int2_t*>(dst) = int2_t{v.x, v.y};
        if (left >= 8) *reinterpret_cast<int2_t*>(dst + 8) = int2_t{v.z, v.w};
    }
}

// What the two forms of the tile function below share: the rows a wave's DMA instructions fetch, a slab's place in
// the ring, what the last iterations of a tile fetch (the "tail"), and the priming of the ring at a tile's start.
// BR x BC outputs per workgroup of NW waves, BKB bytes of K per slab, NST ring stages; LAY / F16 as in the tile functions.
// TSW: a (K, L) operand lands with the units of every row of K exchanged within their 128-byte group -- fp16: unit
// (32 bytes) u of row k at u ^ (k & 3); int8: unit (16 bytes) u at u ^ (k & 7) -- which is what keeps the transposing
// fragment reads free of bank conflicts.  The DMA writes LDS in lane order, so the exchange happens in the choice of
// what a lane fetches.
template <int BR, int BC, int BKB, int NW, int NST, int LAY, bool F16, bool TSW = false>
struct SlabDma {
    static constexpr bool PT = (LAY & 1) != 0, QT = (LAY & 2) != 0;
    static constexpr int ESZ_IN = F16 ? 2 : 1;            // bytes per operand element
    static constexpr int EPP = 16 / ESZ_IN;               // elements per 16-byte piece
    static constexpr int CPR = BKB / 16;                  // 16-byte chunks per row of a slab
    static constexpr int RPW = 256 / BKB;                 // rows per 256-byte bank wrap
    static constexpr int STAGE = (BR + BC) * BKB;
    static constexpr int RPI = 1024 / BKB;                // rows per DMA instruction
    static constexpr int NDMA = (BR + BC) / RPI;
    static_assert(NDMA % NW == 0, "stage must split evenly over the waves");
    static_assert(!TSW || ((BR * ESZ_IN) % 128 == 0 && (BC * ESZ_IN) % 128 == 0), "the exchange of units stays inside whole 128-byte groups of a row of K");
    static constexpr int CNT = NDMA / NW;                 // DMA instructions per wave and slab

    const GemmArgs& a;
    const int wave, lane;
    int nk;                     // slabs per tile
    bool ahead;                 // the next tile is fetched ahead (only if its LDS layout is this one's)
    bool deep;                  // at least as many slabs as stages
    int LD;                     // slabs in flight: the slab requested at iteration `it` is number it + LD of this tile
    int ring0;                  // stage of this tile's slab 0
    int32_t tj0, ti0;           // rows / columns the tail fetches
    const int8_t *Pb, *Qb, *Pn, *Qn;
    uint32_t voff[CNT], ldst[CNT];
    bool isq[CNT];
    int64_t kstepP, kstepQ;     // bytes from one K slab to the next

    __device__ __forceinline__ static int swz(int r) { return (r / RPW) & (CPR - 1); }

    // byte offset of this lane's 16 bytes inside slab 0 of the tile at rows oj / columns oi, for the wave's DMA
    // instruction d -> stage rows [RPI*dd, RPI*dd + RPI), dd = wave + d*NW; rows past the matrix are clamped (they only
    // feed outputs that are never stored)
    __device__ __forceinline__ uint32_t calc_voff(int d, int32_t oj, int32_t oi) const {
        const int dd = wave + d * NW;
        const int r = dd * RPI + lane / CPR;
        const int c = (lane % CPR) ^ swz(r);
        const bool q = dd * RPI >= BR;
        if ((PT && !q) || (QT && q)) {
            // a (K, L) operand: the instruction covers 1024 / (2 * B) rows of K, a lane one 16-byte piece of a row
            const int ppr = (q ? BC : BR) / EPP;                   // pieces per row of K
            const int dl = q ? dd - BR / RPI : dd;
            const int kr = dl * (64 / ppr) + lane / ppr;
            const int pl = lane % ppr;                             // the piece's place in the row of K in LDS
            const int pc = !TSW ? pl : F16 ? ((((pl >> 1) ^ (kr & 3)) << 1) | (pl & 1)) : (pl ^ (kr & 7));      // ... and which piece of the row it is
            const int32_t L = q ? a.m : a.n;
            return ((uint32_t)kr * (uint32_t)L + (uint32_t)min((q ? oi : oj) + pc * EPP, L - EPP)) * (uint32_t)ESZ_IN;      // L % EPP == 0
        }
        const int32_t grow = q ? min(oi + (r - BR), a.m - 1) : min(oj + r, a.n - 1);
        return (uint32_t)grow * (uint32_t)a.k + c * 16;
    }

    __device__ __forceinline__ SlabDma(const GemmArgs& a_, uint32_t lds_base, const GemmItem& cur_item, const GemmItem& nxt_item,
                                       int wave_, int lane_, int ring)
        : a(a_), wave(wave_), lane(lane_) {
        nk = a.k / BKB;
        const uint32_t b = cur_item.b;
        Pb = a.P + (int64_t)b * a.strideP;
        Qb = a.Q + (int64_t)b * a.strideQ;
        ahead = nxt_item.valid && nxt_item.half == cur_item.half;
        // slab s of this tile lives in stage (ring + s) % NST.  With fewer slabs than stages (!deep) all of a
        // tile's slabs are requested one tile ahead and every wait is a full one.
        deep = nk >= NST;
        LD = deep ? NST : nk;
        ring0 = __builtin_amdgcn_readfirstlane(ring);
        // what the last LD iterations fetch: the next tile's first slabs, or (not ahead) this tile's last slab again
        const uint32_t tb = ahead ? nxt_item.b : b;
        tj0 = ahead ? nxt_item.j0 : cur_item.j0;
        ti0 = ahead ? nxt_item.i0 : cur_item.i0;
        Pn = a.P + (int64_t)tb * a.strideP;
        Qn = a.Q + (int64_t)tb * a.strideQ;
#pragma unroll
        for (int d = 0; d < CNT; ++d) {
            const int dd = wave + d * NW;
            isq[d] = dd * RPI >= BR;
            voff[d] = calc_voff(d, cur_item.j0, cur_item.i0);
            ldst[d] = lds_base + dd * 1024;
        }
        kstepP = PT ? (int64_t)BKB * a.n : BKB;
        kstepQ = QT ? (int64_t)BKB * a.m : BKB;
    }

    // One DMA instruction of slab kt into ring stage `stage`: of this tile's rows, or (TAIL) of the rows the last LD
    // iterations fetch -- the next tile's when it is fetched ahead, else this tile's again.  Which one is a
    // compile-time choice: a run-time select here makes the compiler branch inside the K loop, which splits its
    // body and breaks the MFMA/memory interleave.
    template <int d, bool TAIL>
    __device__ __forceinline__ void issue(int kt, int stage) const {
        // read every candidate first and select values, never addresses of the members
        const int8_t *pb = TAIL ? Pn : Pb, *qb = TAIL ? Qn : Qb;
        const uint32_t v = voff[d];            // (rewritten for the tail between the two loops: retarget)
        const bool q = isq[d];
        lds_dma16(v, (q ? qb : pb) + kt * (q ? kstepQ : kstepP), ldst[d] + stage * STAGE);
    }

    // between a tile's main iterations and its tail: the offsets of the rows the tail fetches
    __device__ __forceinline__ void retarget() {
#pragma unroll
        for (int d = 0; d < CNT; ++d) voff[d] = calc_voff(d, tj0, ti0);
    }

    // A tile's start.  Without slabs on their way: request the first NST, wait for slab 0.  Otherwise the first LD
    // slabs were requested during the previous tile; its stores drain too.
    __device__ __forceinline__ void prime(bool have_slabs) const {
        if (!have_slabs) {
            __syncthreads();                 // every wave is done with the ring of the previous tile
            static_for<0, NST>([&](auto sc) __attribute__((always_inline)) {
                constexpr int st = decltype(sc)::value;
                static_for<0, CNT>([&](auto dc) __attribute__((always_inline)) {
                    issue<decltype(dc)::value, false>(min(st, nk - 1), (ring0 + st) % NST);
                });
            });
            if (deep) wait_vmcnt<(NST - 1) * CNT>();   // slab 0 (and the scale loads issued before it) has landed
            else wait_vmcnt<0>();
            __syncthreads();
        } else {
            wait_vmcnt<0>();
            __syncthreads();
        }
    }
};

// The way out of a tile, shared by the two forms of the tile function.  Results leave through a 4 KB strip of
// LDS per wave: a lane holds 4-column pieces of ONE output row, so storing straight from the accumulators
// would touch 32 different rows with 8 or 16 bytes each per instruction.  Written to the strip as 32 rows x RB
// bytes and read back 16 bytes per lane, every store instruction covers whole contiguous rows of the chunk
// (RB = 128 bytes: eight lanes per 128-byte line).
template <int EPI, int TC>
struct StripOut {
    static constexpr int ESZ = EPI == kEpiInt32 ? 4 : 2;
    static constexpr int CT = EPI == kEpiInt32 ? 1 : TC;       // MFMA tile columns (of 32) side by side in one chunk
    static constexpr int NCH = EPI == kEpiInt32 ? TC : 1;      // chunks per block of 32 rows
    static constexpr int RB = CT * 32 * ESZ, PPR = RB / 16, RPW2 = 256 / RB, PASSES = PPR / 2, RPP = 64 / PPR;
    // 16-byte piece p of strip row r sits at piece slot p ^ ((r / RPW2) % PPR): reads are conflict free
    static __device__ __forceinline__ int slot(int r, int p) { return (p ^ ((r / RPW2) & (PPR - 1))) << 4; }
    // the strip's 32 rows go out: output rows row0 .. row0 + 31, columns from col0 on
    static __device__ __forceinline__ void store_rows(const GemmArgs& a, const int8_t* stg, int64_t obase, int32_t row0, int32_t col0, int lane) {
#pragma unroll
        for (int ps = 0; ps < PASSES; ++ps) {
            const int R = ps * RPP + lane / PPR, pc = lane % PPR;
            const int4_t v = *reinterpret_cast<const int4_t*>(stg + R * RB + slot(R, pc));
            const int32_t row = row0 + R;
            const int32_t col = col0 + pc * (16 / ESZ);
            if (row < a.n && col < a.m)
                store_piece<ESZ>(reinterpret_cast<int8_t*>(a.out) + (obase + (int64_t)row * a.m + col) * ESZ, v, a.m - col);
        }
    }
};

// One output tile of BR x BC = (WR*TR*32) x (WC*TC*32), K slab = BKB bytes.
// The MFMA is the 16x16 one with 64 bytes of K (v_mfma_i32_16x16x64_i8, v_mfma_f32_16x16x32_f16):
// per operation it moves half the accumulator registers of the 32x32 form, and on random operands,
// where the chip's power limit sets the clock, the same product finishes about a tenth sooner.
// A wave owns AR x AC = 2TR x 2TC such tiles; lane (r = l % 16, q = l / 16) feeds 16 bytes of K
// (chunk q of the k-step) of row r of each operand block and receives output row r, columns
// 4q .. 4q+3 of each 16x16 tile (the operands are passed swapped).
// A k-step is two passes over the wave's rows, one per half of its columns: the column fragments
// come in two sets, one multiplied while the other is read, and a row fragment's register is
// refilled with the next k-step's right after its last MFMA of the second pass.
// NST-stage ring; pipeline per K slab `it` (stage cur = it % NST, slabs it+1 .. it+NST-1 in flight):
//   k-steps 0 .. KS-2, and the first pass of k-step KS-1 : MFMAs while the fragments that come
//                       next are read from stage cur
//   s_waitcnt vmcnt((NST-2)*CNT); barrier -> slab it+1 has landed in stage nxt for every wave and
//                                      nobody reads stage cur any more
//   second pass of k-step KS-1 : MFMAs while the step-0 fragments of slab it+1 are read and
//                       the DMA of slab it+NST is issued into stage cur
// The last iterations (the "tail", a second copy of the loop body) fetch the first slabs of the
// NEXT tile of this workgroup when it has the same shape, so that tile starts with its operands
// already in LDS and the loads overlap this tile's stores; otherwise they fetch this tile's last
// slab again (a redundant load nobody reads).  The ring position carries over from tile to tile
// (`ring`), so any slab count works.  Each loop body is one basic block without selects, which
// lets the compiler keep the accumulators in place and the MFMA/memory interleave as written.
// Returns true if the next tile's first slabs are on their way.
//
// LAY bit 2: the depth is not whole slabs (any multiple of 4 bytes).  The slabs of the ring cover the whole ones; the
// rest of the depth (less than a slab) goes from memory straight into the fragment registers before the K loop starts
// -- a lane's 16 bytes of a k-step are the same bytes in memory as in the stage -- with zeros past the end of K.  (An
// operand stored (K, rows) beside it: the 32x32 form only, which gathers such a fragment element by element.)
// LAY bit 3, with bit 2: the rest of a row may start off a 16-byte boundary and end inside a piece (depths and rows of
// whole dwords only); without it every piece of the rest is whole and aligned.
// LAY marks operands whose rows are K instead: bit 0 = the row operand is stored (K, n), bit 1 =
// the column operand is stored (K, m).  Such an operand's part of a stage holds the slab's rows
// of K (64 for fp16, 128 for int8) with the tile's BR (BC) elements each, DMA'd as they lie in
// memory (with the units of a row exchanged, SlabDma's TSW); a lane then gets its 16 bytes of K with two
// transposing LDS reads instead of one 16-byte read.
template <int WR, int WC, int TR, int TC, int BKB, int EPI, int NST, int LAY = 0>
__device__ __forceinline__ bool gemm_dma_tile(const GemmArgs& a, int8_t* smem, int8_t* stg, uint32_t lds_base,
                                              const GemmItem cur_item, const GemmItem nxt_item, const bool have_slabs, int& ring) {
    constexpr bool FUSED = EPI == kEpiDequant, F16 = EPI == kEpiF16;
    constexpr bool PT = (LAY & 1) != 0, QT = (LAY & 2) != 0;
    static_assert((LAY & 3) == 0 || BKB == 128, "transposed operands: 128 bytes of K per slab");
    constexpr int ESZ_IN = F16 ? 2 : 1;            // bytes per operand element
    using acc_t = std::conditional_t<F16, float4_t, int4_t>;
    constexpr int KS = BKB / 64, CPR = BKB / 16;
    static_assert(KS >= 1, "k-steps of 64 bytes");
    constexpr int AR = TR * 2, AC = TC * 2;        // 16x16 MFMA tiles of a wave
    constexpr int NW = WR * WC, BR = WR * TR * 32, BC = WC * TC * 32;
    constexpr bool TRP = PT, TRQ = QT;             // fragments of a (K, L) operand: transposing LDS reads
    using Dma = SlabDma<BR, BC, BKB, NW, NST, LAY, F16, TRP || TRQ>;
    constexpr int STAGE = Dma::STAGE, CNT = Dma::CNT;      // bytes per ring stage; DMA instructions per wave and slab
    constexpr int RPW = 256 / BKB;                 // rows per 256-byte bank wrap
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = wave / WC, wc = wave % WC;
    const int r16 = lane & 15, q = lane >> 4;
    const int32_t K = a.k;
    const int nk = K / BKB;
    auto swz = [](int r) __attribute__((always_inline)) { return (r / RPW) & (CPR - 1); };
    // fragment offsets of the wave's first block of 16 rows, k-step 0.  Step s reads logical chunk
    // 4s + q: xor (4s << 4) commutes with the swizzle; block i lies 16 rows further on, where the swizzle repeats.
    static_assert((16 / RPW) % CPR == 0, "the swizzle must repeat every 16 rows");
    constexpr int BLKP = 16 * BKB, BLKQ = 16 * BKB;        // (K-major operands; the others: tr_frag below)
    const int rp0 = wr * TR * 32 + r16, rq0 = wc * TC * 32 + r16;
    const int offP0 = rp0 * BKB + ((q ^ swz(rp0)) << 4);
    const int offQ0 = BR * BKB + rq0 * BKB + ((q ^ swz(rq0)) << 4);
    // without slabs on their way the waits below count only loads: let the previous tile's stores finish first
    if (!have_slabs) wait_vmcnt<0>();
    Dma dma(a, lds_base, cur_item, nxt_item, wave, lane, ring);
    const uint32_t b = cur_item.b;
    const int32_t j0 = cur_item.j0, i0 = cur_item.i0;
    const bool ahead = dma.ahead;
    const int LD = dma.LD, ring0 = dma.ring0;
    auto dma1 = [&](auto dc, int kt, auto tailc, int stage) __attribute__((always_inline)) {
        dma.template issue<decltype(dc)::value, decltype(tailc)::value>(kt, stage);
    };

    // the dequantisation scales of this lane's outputs, fetched now so that the epilogue does
    // not wait on memory between its stores
    half_t sxh[AR];
    half4_t syh[AC];
    if (FUSED) {
#pragma unroll
        for (int i = 0; i < AR; ++i) {
            const int32_t row = min(j0 + wr * TR * 32 + i * 16 + r16, a.n - 1);
            sxh[i] = a.srow[a.bc_row ? row : (int64_t)b * a.n + row];
        }
#pragma unroll
        for (int j = 0; j < AC; ++j) {
            const int32_t col = min(i0 + wc * TC * 32 + j * 16 + q * 4, a.m - 4);   // m % 4 == 0
            syh[j] = *reinterpret_cast<const half4_t*>(a.scol + (a.bc_col ? 0 : (int64_t)b * a.m) + col);
        }
    }

    acc_t acc[AR][AC];
#pragma unroll
    for (int i = 0; i < AR; ++i)
#pragma unroll
        for (int j = 0; j < AC; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[i][j][e] = 0;
    if constexpr ((LAY & 4) != 0) {
        const int32_t K1 = nk * BKB, rem = K - K1;
        if (rem > 0) {
            const int8_t* Pr = a.P + (int64_t)b * a.strideP + K1;
            const int8_t* Qr = a.Q + (int64_t)b * a.strideQ + K1;
            // bytes [kc, kc + 16) of the rest of a row, zeros from byte `rem` on: the piece may start at any address and
            // end inside (rows of K that are whole dwords, not whole 16-byte pieces)
            struct __attribute__((packed, aligned(1))) Piece16 { uint32_t x, y, z, w; };
            // (without branches -- a load under a condition would be waited for before the next one is issued: the 16 bytes
            // that end where the piece or K ends, moved down by the dwords that lie beyond K)
            auto piece = [&](const int8_t* rest, int32_t kc) __attribute__((always_inline)) {
                if constexpr ((LAY & 8) == 0) {      // whole pieces only: one load under one condition
                    int4_t v = {0, 0, 0, 0};
                    if (kc < rem) {
                        const Piece16 t = *reinterpret_cast<const Piece16*>(rest + kc);
                        v = int4_t{(int32_t)t.x, (int32_t)t.y, (int32_t)t.z, (int32_t)t.w};
                    }
                    return v;
                }
                const int32_t over = min(max(kc + 16 - rem, 0), 16);        // bytes of the piece beyond K: 0, 4 ... 16
                const Piece16 t = *reinterpret_cast<const Piece16*>(rest + min(kc - over, rem - 16));       // (inside the row: at least one slab precedes `rest`)
                const int32_t w[8] = {(int32_t)t.x, (int32_t)t.y, (int32_t)t.z, (int32_t)t.w, 0, 0, 0, 0};
                const int sh = over >> 2;
                int4_t v;
#pragma unroll
                for (int d = 0; d < 4; ++d) v[d] = sh == 0 ? w[d] : sh == 1 ? w[d + 1] : sh == 2 ? w[d + 2] : sh == 3 ? w[d + 3] : 0;
                return v;
            };
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                if (ks * 64 < rem) {
                    const int32_t kc = ks * 64 + q * 16;
                    int4_t rp[AR], rq[AC];
#pragma unroll
                    for (int i = 0; i < AR; ++i) rp[i] = piece(Pr + (int64_t)min(j0 + wr * TR * 32 + i * 16 + r16, a.n - 1) * K, kc);
#pragma unroll
                    for (int j = 0; j < AC; ++j) rq[j] = piece(Qr + (int64_t)min(i0 + wc * TC * 32 + j * 16 + r16, a.m - 1) * K, kc);
#pragma unroll
                    for (int i = 0; i < AR; ++i)
#pragma unroll
                        for (int j = 0; j < AC; ++j) {
                            if constexpr (F16)
                                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, rq[j]), __builtin_bit_cast(half8_t, rp[i]), acc[i][j], 0, 0, 0);
                            else
                                acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(rq[j], rp[i], acc[i][j], 0, 0, 0);
                        }
                }
            }
        }
    }
    // Fragments: all AR of the row operand, and the column operand's in two sets of AC/2 -- a k-step is two
    // passes over the wave's rows, one per half of its columns, and while one set is multiplied the
    // other is read.  A row fragment's register is refilled with the next k-step's right after
    // its last MFMA of the second pass.
    constexpr int HC = AC / 2;
    int4_t fp[AR], fq[2][HC];
    // Transposing reads.  fp16 (ds_read_b64_tr_b16): within 16 lanes, lane j hands in the address of four halves -- row
    // of K k0 + j / 4, elements 4 (j % 4) .. + 3 of a block of 16 -- and lane i receives element i of rows k0 .. k0 + 3:
    // four consecutive values of K for its own row of the MFMA operand.  int8 (ds_read_b64_tr_b8): lane j hands in
    // eight bytes -- row of K k0 + j / 2, elements 8 (j % 2) .. + 7 -- and lane i receives element i of rows k0 .. k0 + 7.
    // Two reads per fragment either way, instead of eight 2-byte or sixteen 1-byte ones.  Block u (16 elements) of
    // row k lies at unit u ^ (k & 3) resp. u ^ (k & 7) (SlabDma, TSW): an exclusive-or of the block's offset with a
    // lane's constant.
    constexpr int ULOG = F16 ? 5 : 4;              // log2 of a block's bytes
    const int trx = F16 ? (r16 >> 2) << 5 : (r16 >> 1) << 4;                  // the exchange, as an offset
    const int trb = F16 ? (r16 & 3) << 3 : (r16 & 1) << 3;                    // the lane's eight bytes within the block
    const int trk = F16 ? q * 8 + (r16 >> 2) : q * 16 + (r16 >> 1);            // the row of K (within a k-step) this lane's first address names
    auto tr_frag = [&](const int8_t* part, int rowlen, int ublock, int ks) __attribute__((always_inline)) {
        // part: the operand's rows of K in the stage; rowlen: bytes per row of K; ublock: number of the block of 16 elements
        const uint32_t p0 = lds_base + (uint32_t)(part - smem) + (ks * (F16 ? 32 : 64) + trk) * rowlen + ((ublock << ULOG) ^ trx) + trb;
        const uint32_t p1 = p0 + (F16 ? 4 : 8) * rowlen;
        if constexpr (F16) {
            typedef short short4_t __attribute__((ext_vector_type(4)));
            const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4_t*)(uintptr_t)p0);
            const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4_t*)(uintptr_t)p1);
            return __builtin_bit_cast(int4_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        } else {
            typedef int int2_tv __attribute__((ext_vector_type(2)));
            const int2_tv lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) int2_tv*)(uintptr_t)p0);
            const int2_tv hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) int2_tv*)(uintptr_t)p1);
            return int4_t{lo.x, lo.y, hi.x, hi.y};
        }
    };
    auto lfragP = [&](auto ic, int stage, int ks) __attribute__((always_inline)) {
        constexpr int i = decltype(ic)::value;
        if constexpr (TRP) fp[i] = tr_frag(smem + stage * STAGE, BR * ESZ_IN, wr * TR * 2 + i, ks);
        else fp[i] = *reinterpret_cast<const int4_t*>(smem + stage * STAGE + (offP0 ^ (ks << 6)) + i * BLKP);
    };
    auto lfragQ = [&](auto setc, auto jjc, int stage, int ks) __attribute__((always_inline)) {       // fragment jj of column half `set`
        constexpr int set = decltype(setc)::value, jj = decltype(jjc)::value;
        constexpr int j = set * HC + jj;
        if constexpr (TRQ) fq[set][jj] = tr_frag(smem + stage * STAGE + BR * BKB, BC * ESZ_IN, wc * TC * 2 + j, ks);
        else fq[set][jj] = *reinterpret_cast<const int4_t*>(smem + stage * STAGE + (offQ0 ^ (ks << 6)) + j * BLKQ);
    };
    // One pass: the AR x HC MFMAs of column half `jh`, order pinned.  Between them the other set of column
    // fragments is read from k-step `qks` of stage `qs`; with REFILL the row fragments are refilled from
    // k-step `nks` of stage `ns`; and ND further memory operations (`memop`) are spread over the pass.
    constexpr int NMP = AR * HC;
    auto pass = [&](auto jhc, int qs, int qks, auto refillc, int ns, int nks, auto&& memop, auto nd_c) __attribute__((always_inline)) {
        constexpr int jh = decltype(jhc)::value, ND = decltype(nd_c)::value;
        constexpr bool REFILL = decltype(refillc)::value;
        static_for<0, NMP>([&](auto xc) __attribute__((always_inline)) {
            constexpr int x = decltype(xc)::value;
            constexpr int i = x / HC, jj = x % HC;
            // MFMA "A" = column-operand rows, "B" = row-operand rows: lane l, register e of the
            // result is output row l%16, column (l/16)*4 + e of the 16x16 tile
            if constexpr (F16)      // 64 bytes of K are 32 halves: same lane -> byte assignment as the int8 MFMA
                acc[i][jh * HC + jj] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, fq[jh][jj]),
                                                                              __builtin_bit_cast(half8_t, fp[i]), acc[i][jh * HC + jj], 0, 0, 0);
            else
                acc[i][jh * HC + jj] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fq[jh][jj], fp[i], acc[i][jh * HC + jj], 0, 0, 0);
            if constexpr (REFILL && jj == HC - 1) lfragP(std::integral_constant<int, i>{}, ns, nks);
            if constexpr (x % AR == 0 && x / AR < HC)
                lfragQ(std::integral_constant<int, 1 - jh>{}, std::integral_constant<int, x / AR>{}, qs, qks);
            constexpr int lo = (x * ND) / NMP, hi = ((x + 1) * ND) / NMP;
            static_for<lo, hi>([&](auto yc) __attribute__((always_inline)) { memop(yc); });
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    auto no_memop = [](auto) __attribute__((always_inline)) {};

    dma.prime(have_slabs);
    if (FUSED) {     // pin the scale loads above the K loop (the waits just above cover them)
#pragma unroll
        for (int i = 0; i < AR; ++i) asm volatile("" : "+v"(sxh[i]));
#pragma unroll
        for (int j = 0; j < AC; ++j) asm volatile("" : "+v"(syh[j]));
        // parked in this wave's output strip, idle until the epilogue: fewer registers live across the K loop
#pragma unroll
        for (int i = 0; i < AR; ++i) *reinterpret_cast<half_t*>(stg + (i * 64 + lane) * 2) = sxh[i];
#pragma unroll
        for (int j = 0; j < AC; ++j) *reinterpret_cast<half4_t*>(stg + 1024 + (j * 64 + lane) * 8) = syh[j];
    }
    static_for<0, AR>([&](auto xc) __attribute__((always_inline)) { lfragP(xc, ring0, 0); });
    static_for<0, HC>([&](auto xc) __attribute__((always_inline)) { lfragQ(I0{}, xc, ring0, 0); });

    int cur = ring0;
    // tail slab index: it + LD - nk of the next tile, or nk - 1 of this one
    const int tmul = ahead ? 1 : 0, tadd = ahead ? LD - nk : nk - 1;
    auto slab = [&](int it, auto tailc) __attribute__((always_inline)) {
        constexpr bool TAIL = decltype(tailc)::value;
        const int nxt = cur + 1 == NST ? 0 : cur + 1;
        static_for<0, KS - 1>([&](auto ksc) __attribute__((always_inline)) {
            constexpr int ks = decltype(ksc)::value;
            pass(I0{}, cur, ks, std::false_type{}, 0, 0, no_memop, I0{});
            pass(I1{}, cur, ks + 1, std::true_type{}, cur, ks + 1, no_memop, I0{});
        });
        pass(I0{}, cur, KS - 1, std::false_type{}, 0, 0, no_memop, I0{});       // the last reads of stage cur
        __builtin_amdgcn_sched_barrier(0);
        wait_vmcnt<(NST - 2) * CNT>();       // slab it + 1 has landed (with fewer slabs than stages it had before the loop)
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        const int kt2 = TAIL ? it * tmul + tadd : it + LD;
        const int tgt = cur + LD >= NST ? cur + LD - NST : cur + LD;       // the stage slab it + LD belongs to
        pass(I1{}, nxt, 0, std::true_type{}, nxt, 0,
             [&](auto dc) __attribute__((always_inline)) { dma1(dc, kt2, tailc, tgt); },
             std::integral_constant<int, CNT>{});
        __builtin_amdgcn_sched_barrier(0);
        cur = nxt;
    };
    int it = 0;
    for (; it < nk - LD; ++it) slab(it, std::false_type{});       // slabs LD .. nk-1 of this tile follow
    dma.retarget();
    for (; it < nk; ++it) slab(it, std::true_type{});             // then the tail's
    if (!ahead) wait_vmcnt<0>();         // drain the clamped loads before the ring is reused
    ring = cur;                          // (ring0 + nk) % NST: where the next tile's slab 0 is, or will be put

    const int64_t obase = (int64_t)b * a.n * a.m;
    using Out = StripOut<EPI, TC>;       // the results leave through this wave's strip of LDS
    constexpr int NCH = Out::NCH, RB = Out::RB;
    auto slot = [](int r, int p) __attribute__((always_inline)) { return Out::slot(r, p); };
    half_t sxr[AR];
    half4_t syr[AC];
    if (FUSED) {      // the scales come back from the strip before the results overwrite it
#pragma unroll
        for (int i = 0; i < AR; ++i) sxr[i] = *reinterpret_cast<const half_t*>(stg + (i * 64 + lane) * 2);
#pragma unroll
        for (int j = 0; j < AC; ++j) syr[j] = *reinterpret_cast<const half4_t*>(stg + 1024 + (j * 64 + lane) * 8);
#pragma unroll
        for (int i = 0; i < AR; ++i) asm volatile("" : "+v"(sxr[i]));
#pragma unroll
        for (int j = 0; j < AC; ++j) asm volatile("" : "+v"(syr[j]));
    }
#pragma unroll
    for (int i = 0; i < TR; ++i) {        // blocks of 32 output rows: two rows of MFMA tiles
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int srow = h * 16 + r16;      // row of the strip
                if constexpr (EPI == kEpiInt32) {
#pragma unroll
                    for (int jj = 0; jj < 2; ++jj)
                        *reinterpret_cast<int4_t*>(stg + srow * RB + slot(srow, jj * 4 + q)) = acc[2 * i + h][2 * c + jj];
                } else {
                    float sx = 0.0f;
                    if (FUSED) sx = (float)sxr[2 * i + h];
#pragma unroll
                    for (int j = 0; j < AC; ++j) {
                        half4_t hv;
                        if constexpr (F16) {
#pragma unroll
                            for (int e = 0; e < 4; ++e) hv[e] = (half_t)acc[2 * i + h][j][e];
                        } else {
                            const half4_t sy = syr[j];
#pragma unroll
                            for (int e = 0; e < 4; ++e) hv[e] = dequant(acc[2 * i + h][j][e], sx, (float)sy[e]);
                        }
                        *reinterpret_cast<half4_t*>(stg + srow * RB + slot(srow, j * 2 + (q >> 1)) + (q & 1) * 8) = hv;
                    }
                }
            }
            Out::store_rows(a, stg, obase, j0 + wr * TR * 32 + i * 32, i0 + wc * TC * 32 + c * 32, lane);
        }
    }
    return ahead;
}

// The same tile with v_mfma_i32_32x32x32_i8 / v_mfma_f32_32x32x16_f16 (k-steps of 32 bytes, a wave owns
// TR x TC tiles of 32x32, lane l holds output row l%32; both operands' fragments double buffered,
// the barrier before the last k-step).  Used where a wave's share of a k-step is too small for the
// row fragments' refill-after-last-use above to hide the LDS latency (the 128x128 and smaller
// workgroup tiles, one wave per SIMD) and for products of a single slab.  DMA, ring and tail are
// the ones described above.
template <int WR, int WC, int TR, int TC, int BKB, int EPI, int NST, int LAY = 0>
__device__ __forceinline__ bool gemm_dma_tile32(const GemmArgs& a, int8_t* smem, int8_t* stg, uint32_t lds_base,
                                              const GemmItem cur_item, const GemmItem nxt_item, const bool have_slabs, int& ring) {
    constexpr bool FUSED = EPI == kEpiDequant, F16 = EPI == kEpiF16;
    constexpr bool PT = (LAY & 1) != 0, QT = (LAY & 2) != 0;
    static_assert((LAY & 3) == 0 || BKB == 128, "transposed operands: 128 bytes of K per slab");
    constexpr int ESZ_IN = F16 ? 2 : 1;            // bytes per operand element
    using acc_t = std::conditional_t<F16, float16_tv, int16_tv>;
    constexpr int KS = BKB / 32, CPR = BKB / 16;
    constexpr int NW = WR * WC, BR = WR * TR * 32, BC = WC * TC * 32;
    constexpr bool TRP = PT, TRQ = QT;             // fragments of a (K, L) operand: transposing LDS reads
    using Dma = SlabDma<BR, BC, BKB, NW, NST, LAY, F16, TRP || TRQ>;
    constexpr int STAGE = Dma::STAGE, CNT = Dma::CNT;      // bytes per ring stage; DMA instructions per wave and slab
    constexpr int NM = TR * TC;
    constexpr int RPW = 256 / BKB;                 // rows per 256-byte bank wrap
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = wave / WC, wc = wave % WC;
    const int lrow = lane & 31, lk = lane >> 5;
    const int32_t K = a.k;
    const int nk = K / BKB;
    auto swz = [](int r) __attribute__((always_inline)) { return (r / RPW) & (CPR - 1); };
    // fragment offsets for k-step 0; step s reads logical chunk 2s + lk: xor (2s << 4) commutes with the swizzle
    int offP[TR], offQ[TC];
#pragma unroll
    for (int i = 0; i < TR; ++i) {
        const int r = wr * TR * 32 + i * 32 + lrow;
        offP[i] = r * BKB + ((lk ^ swz(r)) << 4);          // (K-major operands; the others: tr_frag below)
    }
#pragma unroll
    for (int j = 0; j < TC; ++j) {
        const int r = wc * TC * 32 + j * 32 + lrow;
        offQ[j] = BR * BKB + r * BKB + ((lk ^ swz(r)) << 4);
    }
    // without slabs on their way the waits below count only loads: let the previous tile's stores finish first
    if (!have_slabs) wait_vmcnt<0>();
    Dma dma(a, lds_base, cur_item, nxt_item, wave, lane, ring);
    const uint32_t b = cur_item.b;
    const int32_t j0 = cur_item.j0, i0 = cur_item.i0;
    const bool ahead = dma.ahead;
    const int LD = dma.LD, ring0 = dma.ring0;
    auto dma1 = [&](auto dc, int kt, auto tailc, int stage) __attribute__((always_inline)) {
        dma.template issue<decltype(dc)::value, decltype(tailc)::value>(kt, stage);
    };

    // the dequantisation scales of this lane's outputs, fetched now so that the epilogue does
    // not wait on memory between its stores
    half_t sxh[TR];
    half4_t syh[TC][4];
    if (FUSED) {
#pragma unroll
        for (int i = 0; i < TR; ++i) {
            const int32_t row = min(j0 + wr * TR * 32 + i * 32 + lrow, a.n - 1);
            sxh[i] = a.srow[a.bc_row ? row : (int64_t)b * a.n + row];
        }
#pragma unroll
        for (int j = 0; j < TC; ++j)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const int32_t col = min(i0 + wc * TC * 32 + j * 32 + g4 * 8 + lk * 4, a.m - 4);   // m % 4 == 0
                syh[j][g4] = *reinterpret_cast<const half4_t*>(a.scol + (a.bc_col ? 0 : (int64_t)b * a.m) + col);
            }
    }

    acc_t acc[TR][TC];
#pragma unroll
    for (int i = 0; i < TR; ++i)
#pragma unroll
        for (int j = 0; j < TC; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;
    if constexpr ((LAY & 4) != 0) {
        // The depth beyond the last whole slab, as in the 16x16 form.  Here either operand may also be stored (K, rows): its
        // fragment -- a lane's 8 (fp16) or 16 (int8) consecutive values of K for its own row -- is then gathered element
        // by element, adjacent lanes reading adjacent elements of a row of K.  K-major pieces may start at any address
        // and end inside the piece (rows of K that are whole dwords, not whole 16-byte pieces).
        const int32_t K1 = nk * BKB, rem = K - K1;           // bytes
        if (rem > 0) {
            constexpr int EPP = 16 / ESZ_IN;
            struct __attribute__((packed, aligned(1))) Piece16 { uint32_t x, y, z, w; };
            const int8_t* Pr = a.P + (int64_t)b * a.strideP;
            const int8_t* Qr = a.Q + (int64_t)b * a.strideQ;
            // a K-major operand's piece: bytes [kc, kc + 16) of the rest of row `row`, zeros from byte `rem` on
            // (both without branches -- a load under a condition would be waited for before the next one is issued.  The
            // piece: the 16 bytes that end where the piece or K ends, moved down by the dwords that lie beyond K.)
            auto piece = [&](const int8_t* base, int32_t row, int32_t kc) __attribute__((always_inline)) {
                if constexpr ((LAY & 8) == 0) {      // whole pieces only: one load under one condition (15 % quicker than the form below where it applies)
                    int4_t v = {0, 0, 0, 0};
                    if (kc < rem) {
                        const Piece16 t = *reinterpret_cast<const Piece16*>(base + (int64_t)row * K + K1 + kc);
                        v = int4_t{(int32_t)t.x, (int32_t)t.y, (int32_t)t.z, (int32_t)t.w};
                    }
                    return v;
                }
                const int32_t over = min(max(kc + 16 - rem, 0), 16);        // bytes of the piece beyond K: 0, 4 ... 16
                const Piece16 t = *reinterpret_cast<const Piece16*>(base + (int64_t)row * K + K1 + min(kc - over, rem - 16));      // (inside the row: at least one slab precedes)
                const int32_t w[8] = {(int32_t)t.x, (int32_t)t.y, (int32_t)t.z, (int32_t)t.w, 0, 0, 0, 0};
                const int sh = over >> 2;
                int4_t v;
#pragma unroll
                for (int d = 0; d < 4; ++d) v[d] = sh == 0 ? w[d] : sh == 1 ? w[d + 1] : sh == 2 ? w[d + 2] : sh == 3 ? w[d + 3] : 0;
                return v;
            };
            // a (K, L) operand's piece: elements [ke, ke + EPP) of the rest of K for element `row` of the rows of K
            auto gather = [&](const int8_t* base, int32_t L, int32_t row, int32_t ke) __attribute__((always_inline)) {
                const int32_t kel0 = K1 / ESZ_IN, krem = rem / ESZ_IN;
                if constexpr (F16) {
                    half8_t h;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const half_t x = reinterpret_cast<const half_t*>(base)[(int64_t)(kel0 + min(ke + e, krem - 1)) * L + row];
                        h[e] = ke + e < krem ? x : (half_t)0.0f;
                    }
                    return __builtin_bit_cast(int4_t, h);
                } else {
                    int4_t v = {0, 0, 0, 0};
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const uint32_t x = (uint8_t)base[(int64_t)(kel0 + min(ke + e, krem - 1)) * L + row];
                        v[e >> 2] |= (int32_t)((ke + e < krem ? x : 0u) << (8 * (e & 3)));
                    }
                    return v;
                }
            };
            auto load_ks = [&](int4_t (&rp)[TR], int4_t (&rq)[TC], int ks) __attribute__((always_inline)) {
                const int32_t kc = ks * 32 + lk * 16;
#pragma unroll
                for (int i = 0; i < TR; ++i) {
                    const int32_t row = min(j0 + wr * TR * 32 + i * 32 + lrow, a.n - 1);
                    rp[i] = int4_t{0, 0, 0, 0};
                    if (ks * 32 < rem) {
                        if constexpr (PT) rp[i] = gather(Pr, a.n, row, kc / ESZ_IN);
                        else rp[i] = piece(Pr, row, kc);
                    }
                }
#pragma unroll
                for (int j = 0; j < TC; ++j) {
                    const int32_t col = min(i0 + wc * TC * 32 + j * 32 + lrow, a.m - 1);
                    rq[j] = int4_t{0, 0, 0, 0};
                    if (ks * 32 < rem) {
                        if constexpr (QT) rq[j] = gather(Qr, a.m, col, kc / ESZ_IN);
                        else rq[j] = piece(Qr, col, kc);
                    }
                }
            };
            auto mac_ks = [&](const int4_t (&rp)[TR], const int4_t (&rq)[TC], int ks) __attribute__((always_inline)) {
                if (ks * 32 < rem) {
#pragma unroll
                    for (int i = 0; i < TR; ++i)
#pragma unroll
                        for (int j = 0; j < TC; ++j) {
                            if constexpr (F16)
                                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, rq[j]), __builtin_bit_cast(half8_t, rp[i]), acc[i][j], 0, 0, 0);
                            else
                                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(rq[j], rp[i], acc[i][j], 0, 0, 0);
                        }
                }
            };
            if constexpr (PT || QT) {
                // gathered fragments are many small loads: every k-step's are requested before the first product -- one trip
                // to memory, not one per k-step
                int4_t rp[KS][TR], rq[KS][TC];
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) load_ks(rp[ks], rq[ks], ks);
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) mac_ks(rp[ks], rq[ks], ks);
            } else {
                // (K-major operands only: a k-step at a time, which keeps the wide accumulator tiles of this form in registers)
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    int4_t rp[TR], rq[TC];
                    load_ks(rp, rq, ks);
                    mac_ks(rp, rq, ks);
                }
            }
        }
    }
    int4_t fp[2][TR], fq[2][TC];
    // Transposing reads as in the 16x16 form.  Here a fragment is 32 rows x 16 bytes of K: the wave's four groups of
    // 16 lanes are (rows 0-15 | 16-31) x (first | second half of the k-step's 32 bytes), so a group's block of 16
    // rows is number 2 i + (group & 1) of the wave's, and its rows of K start at 8 (fp16) or 16 (int8) times group >> 1.
    constexpr int ULOG = F16 ? 5 : 4;              // log2 of a block's bytes
    const int trj = lane & 15, trg = lane >> 4;
    const int trx = F16 ? (trj >> 2) << 5 : (trj >> 1) << 4;                  // the exchange, as an offset
    const int trb = F16 ? (trj & 3) << 3 : (trj & 1) << 3;                    // the lane's eight bytes within the block
    const int trk = F16 ? (trg >> 1) * 8 + (trj >> 2) : (trg >> 1) * 16 + (trj >> 1);      // the row of K (within a k-step) of the lane's first address
    auto tr_frag = [&](const int8_t* part, int rowlen, int ublock0, auto ic, int ks) __attribute__((always_inline)) {
        // part: the operand's rows of K in the stage; rowlen: bytes per row of K; ublock0: number of the wave's first block of 16 elements
        constexpr int i = decltype(ic)::value;
        const uint32_t p0 = lds_base + (uint32_t)(part - smem) + (ks * (F16 ? 16 : 32) + trk) * rowlen + (((ublock0 + 2 * i + (trg & 1)) << ULOG) ^ trx) + trb;
        const uint32_t p1 = p0 + (F16 ? 4 : 8) * rowlen;
        if constexpr (F16) {
            typedef short short4_t __attribute__((ext_vector_type(4)));
            const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4_t*)(uintptr_t)p0);
            const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4_t*)(uintptr_t)p1);
            return __builtin_bit_cast(int4_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        } else {
            typedef int int2_tv __attribute__((ext_vector_type(2)));
            const int2_tv lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) int2_tv*)(uintptr_t)p0);
            const int2_tv hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) int2_tv*)(uintptr_t)p1);
            return int4_t{lo.x, lo.y, hi.x, hi.y};
        }
    };
    auto lfrag1 = [&](auto xc, auto bufc, int stage, int ks) __attribute__((always_inline)) {
        constexpr int x = decltype(xc)::value, buf = decltype(bufc)::value;
        if constexpr (x < TR) {
            if constexpr (TRP) {
                fp[buf][x] = tr_frag(smem + stage * STAGE, BR * ESZ_IN, wr * TR * 2, std::integral_constant<int, x>{}, ks);
            } else {
                fp[buf][x] = *reinterpret_cast<const int4_t*>(smem + stage * STAGE + (offP[x] ^ (ks << 5)));
            }
        } else {
            if constexpr (TRQ) {
                fq[buf][x - TR] = tr_frag(smem + stage * STAGE + BR * BKB, BC * ESZ_IN, wc * TC * 2, std::integral_constant<int, x - TR>{}, ks);
            } else {
                fq[buf][x - TR] = *reinterpret_cast<const int4_t*>(smem + stage * STAGE + (offQ[x - TR] ^ (ks << 5)));
            }
        }
    };
    // one k-step: NM MFMAs with NMEM memory operations spread evenly between them, order pinned
    auto kstep = [&](auto bufc, auto&& memop, auto nmem_c) __attribute__((always_inline)) {
        constexpr int NMEM = decltype(nmem_c)::value, buf = decltype(bufc)::value;
        static_for<0, NM>([&](auto xc) __attribute__((always_inline)) {
            constexpr int x = decltype(xc)::value;
            constexpr int i = x / TC, j = x % TC;
            // MFMA "A" = column-operand rows, "B" = row-operand rows: lane l, register e of the
            // result is output row l%32, column (e/4)*8 + (l/32)*4 + e%4 of the 32x32 tile
            if constexpr (F16)      // 32 bytes of K are 16 halves: same lane -> byte assignment as the int8 MFMA
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, fq[buf][j]),
                                                                   __builtin_bit_cast(half8_t, fp[buf][i]), acc[i][j], 0, 0, 0);
            else
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fq[buf][j], fp[buf][i], acc[i][j], 0, 0, 0);
            constexpr int lo = (x * NMEM) / NM, hi = ((x + 1) * NMEM) / NM;
            static_for<lo, hi>([&](auto yc) __attribute__((always_inline)) { memop(yc); });
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    using C0 = std::integral_constant<int, 0>;

    dma.prime(have_slabs);
    if (FUSED) {     // pin the scale loads above the K loop (the waits just above cover them)
#pragma unroll
        for (int i = 0; i < TR; ++i) asm volatile("" : "+v"(sxh[i]));
#pragma unroll
        for (int j = 0; j < TC; ++j)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) asm volatile("" : "+v"(syh[j][g4]));
        // parked in this wave's output strip, idle until the epilogue: 20 fewer registers live across the K loop
#pragma unroll
        for (int i = 0; i < TR; ++i) *reinterpret_cast<half_t*>(stg + (i * 64 + lane) * 2) = sxh[i];
#pragma unroll
        for (int j = 0; j < TC; ++j)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) *reinterpret_cast<half4_t*>(stg + 1024 + lk * 64 + (j * 4 + g4) * 8) = syh[j][g4];
    }
    static_for<0, TR + TC>([&](auto xc) __attribute__((always_inline)) { lfrag1(xc, C0{}, ring0, 0); });

    int cur = ring0;
    // tail slab index: it + LD - nk of the next tile, or nk - 1 of this one
    const int tmul = ahead ? 1 : 0, tadd = ahead ? LD - nk : nk - 1;
    auto slab = [&](int it, auto tailc) __attribute__((always_inline)) {
        constexpr bool TAIL = decltype(tailc)::value;
        const int nxt = cur + 1 == NST ? 0 : cur + 1;
        static_for<0, KS - 1>([&](auto ksc) __attribute__((always_inline)) {
            constexpr int ks = decltype(ksc)::value;
            kstep(std::integral_constant<int, (ks & 1)>{},
                  [&](auto xc) __attribute__((always_inline)) {
                      lfrag1(xc, std::integral_constant<int, ((ks + 1) & 1)>{}, cur, ks + 1);
                  },
                  std::integral_constant<int, TR + TC>{});
        });
        __builtin_amdgcn_sched_barrier(0);
        wait_vmcnt<(NST - 2) * CNT>();       // slab it + 1 has landed (with fewer slabs than stages it had before the loop)
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        const int kt2 = TAIL ? it * tmul + tadd : it + LD;
        const int tgt = cur + LD >= NST ? cur + LD - NST : cur + LD;       // the stage slab it + LD belongs to
        kstep(std::integral_constant<int, ((KS - 1) & 1)>{},
              [&](auto xc) __attribute__((always_inline)) {
                  constexpr int x = decltype(xc)::value;
                  if constexpr (x < TR + TC) lfrag1(xc, std::integral_constant<int, (KS & 1)>{}, nxt, 0);
                  else dma1(std::integral_constant<int, x - (TR + TC)>{}, kt2, tailc, tgt);
              },
              std::integral_constant<int, TR + TC + CNT>{});
        __builtin_amdgcn_sched_barrier(0);
        cur = nxt;
    };
    int it = 0;
    for (; it < nk - LD; ++it) slab(it, std::false_type{});       // slabs LD .. nk-1 of this tile follow
    dma.retarget();
    for (; it < nk; ++it) slab(it, std::true_type{});             // then the tail's
    if (!ahead) wait_vmcnt<0>();         // drain the clamped loads before the ring is reused
    ring = cur;                          // (ring0 + nk) % NST: where the next tile's slab 0 is, or will be put

    const int64_t obase = (int64_t)b * a.n * a.m;
    using Out = StripOut<EPI, TC>;       // the results leave through this wave's strip of LDS
    constexpr int NCH = Out::NCH, RB = Out::RB;
    auto slot = [](int r, int p) __attribute__((always_inline)) { return Out::slot(r, p); };
    half_t sxr[TR];
    half4_t syr[TC][4];
    if (FUSED) {      // the scales come back from the strip before the results overwrite it
#pragma unroll
        for (int i = 0; i < TR; ++i) sxr[i] = *reinterpret_cast<const half_t*>(stg + (i * 64 + lane) * 2);
#pragma unroll
        for (int j = 0; j < TC; ++j)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) syr[j][g4] = *reinterpret_cast<const half4_t*>(stg + 1024 + lk * 64 + (j * 4 + g4) * 8);
#pragma unroll
        for (int i = 0; i < TR; ++i) asm volatile("" : "+v"(sxr[i]));
#pragma unroll
        for (int j = 0; j < TC; ++j)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) asm volatile("" : "+v"(syr[j][g4]));
    }
#pragma unroll
    for (int i = 0; i < TR; ++i) {
        float sx = 0.0f;
        if (FUSED) sx = (float)sxr[i];
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            if constexpr (EPI == kEpiInt32) {
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    const int4_t v = {(int32_t)acc[i][c][g4 * 4], (int32_t)acc[i][c][g4 * 4 + 1],
                                      (int32_t)acc[i][c][g4 * 4 + 2], (int32_t)acc[i][c][g4 * 4 + 3]};
                    *reinterpret_cast<int4_t*>(stg + lrow * RB + slot(lrow, g4 * 2 + lk)) = v;
                }
            } else {
#pragma unroll
                for (int j = 0; j < TC; ++j)
#pragma unroll
                    for (int g4 = 0; g4 < 4; ++g4) {
                        half4_t h;
                        if constexpr (F16) {
#pragma unroll
                            for (int e = 0; e < 4; ++e) h[e] = (half_t)acc[i][j][g4 * 4 + e];
                        } else {
                            const half4_t sy = syr[j][g4];
#pragma unroll
                            for (int e = 0; e < 4; ++e) h[e] = dequant(acc[i][j][g4 * 4 + e], sx, (float)sy[e]);
                        }
                        *reinterpret_cast<half4_t*>(stg + lrow * RB + slot(lrow, j * 4 + g4) + lk * 8) = h;
                    }
            }
            Out::store_rows(a, stg, obase, j0 + wr * TR * 32 + i * 32, i0 + wc * TC * 32 + c * 32, lane);
        }
    }
    return ahead;
}

// Persistent kernel: WR x WC waves, wave tile = TR x TC blocks of 32x32 outputs, computed with the
// 16x16 MFMAs (MF = 16) or the 32x32 ones (MF = 32).  Workgroup w of G
// takes items round*G + (w%8)*(G/8) + w/8: the workgroups of one XCD (w % 8) work on adjacent
// tiles and share operand slabs in that XCD's L2.  When the tile count leaves a last round
// that at most half the workgroups could join, those tiles are issued as row halves (HALVES), one
// per workgroup: a wave then owns TR/2 x TC blocks, which keeps the fragment reads per MFMA
// lower than halving the columns would.
template <int WR, int WC, int TR, int TC, int BKB, int EPI, bool HALVES, int NST, int LAY, int MF>
__global__ __launch_bounds__(WR* WC * 64) void k_gemm_dma(DmaArgs da) {
    static_assert(!(HALVES && LAY != 0), "half tiles only with K-major operands");
    static_assert(MF == 16 || MF == 32, "MFMA tile");
    constexpr int BR = WR * TR * 32, BC = WC * TC * 32;
    extern __shared__ __attribute__((aligned(16))) int8_t smem[];
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) int8_t*)smem;
    // behind the operand ring: one 4 KB strip per wave for the output rows on their way out
    constexpr int STRIP = TC * 64 * 32 > 4096 ? TC * 64 * 32 : 4096;      // 32 rows of the widest chunk (fp16: TC*64 bytes, int32: 128)
    int8_t* stg = smem + NST * (BR + BC) * BKB + (threadIdx.x >> 6) * STRIP;
    const uint32_t G = gridDim.x;
    const uint32_t w = (G % 8 == 0) ? (blockIdx.x % 8) * (G / 8) + blockIdx.x / 8 : blockIdx.x;
    bool have_slabs = false;
    int ring = 0;
    GemmItem cur = gemm_item<BR, BC>(w, da);
    for (uint32_t L = w; cur.valid; L += G) {
        const GemmItem nxt = gemm_item<BR, BC>(L + G, da);
        if (HALVES && cur.half) {
            if constexpr (HALVES) {
                if constexpr (MF == 16) have_slabs = gemm_dma_tile<WR, WC, TR / 2, TC, BKB, EPI, NST>(da.g, smem, stg, lds_base, cur, nxt, have_slabs, ring);
                else have_slabs = gemm_dma_tile32<WR, WC, TR / 2, TC, BKB, EPI, NST>(da.g, smem, stg, lds_base, cur, nxt, have_slabs, ring);
            }
        } else {
            if constexpr (MF == 16) have_slabs = gemm_dma_tile<WR, WC, TR, TC, BKB, EPI, NST, LAY>(da.g, smem, stg, lds_base, cur, nxt, have_slabs, ring);
            else have_slabs = gemm_dma_tile32<WR, WC, TR, TC, BKB, EPI, NST, LAY>(da.g, smem, stg, lds_base, cur, nxt, have_slabs, ring);
        }
        cur = nxt;
    }
}

// ---------------------------------------------------------------------------------------
// Generic path: 64x64 output tile, 32 bytes of K per stage, 256 threads each computing a
// 4x4 block with v_dot4_i32_i8.  Element-wise guarded loads handle every layout and size.
// ---------------------------------------------------------------------------------------
template <bool FUSED>
__global__ __launch_bounds__(256) void k_gemm_generic(GemmArgs a, int p_kmajor, int q_kmajor, int32_t row_base) {
    constexpr int T = 64, GK = 32, LD = GK + 4;
    __shared__ __attribute__((aligned(4))) int8_t sP[T * LD];
    __shared__ __attribute__((aligned(4))) int8_t sQ[T * LD];
    const int b = blockIdx.z;
    const int8_t* P = a.P + (int64_t)b * a.strideP;
    const int8_t* Q = a.Q + (int64_t)b * a.strideQ;
    const int32_t j0 = row_base + blockIdx.y * T, i0 = blockIdx.x * T;
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

template <int WAVES_R, int WAVES_C, int TR, int TC, bool FUSED, bool DW = false>
static int launch_kmajor(GemmArgs& a, int batch, hipStream_t st) {
    constexpr int BR = WAVES_R * TR * 32, BC = WAVES_C * TC * 32;
    constexpr int smem = 2 * (BR + BC) * BK;
    a.tiles_r = (int32_t)ceil_div(a.n, BR);
    a.tiles_c = (int32_t)ceil_div(a.m, BC);
    auto kern = k_gemm_kmajor<WAVES_R, WAVES_C, TR, TC, FUSED, DW>;
    static std::atomic<bool> lds_enabled[64];
    if (smem > 48 * 1024)
        if (int e = enable_dynamic_lds(reinterpret_cast<const void*>(kern), smem, lds_enabled)) return e;
    dim3 grid((unsigned)(a.tiles_r * a.tiles_c), 1, (unsigned)batch);
    hipLaunchKernelGGL(kern, grid, dim3(WAVES_R * WAVES_C * 64), smem, st, a);
    return launch_status();
}

// Ring stages: four for the 128x128 and 128x64 tile kernels, which finish a slab before a load from L2 returns (two, three,
// six and eight stages, and slabs of 64 or 256 bytes, all measured 1-3 us slower at 512 x 4096 x 4096); two for the
// 256x256 tile, whose ring then fills the LDS beside the output strips.
constexpr int kRingSmall = 4, kRingBig = 2;

template <int WR, int WC, int TR, int TC, int BKB, int EPI, bool HALVES, int NST, int LAY, int MF>
static int launch_dma_kernel(const DmaArgs& da, unsigned grid, hipStream_t st) {
    constexpr int BR = WR * TR * 32, BC = WC * TC * 32;
    constexpr int STRIP = TC * 64 * 32 > 4096 ? TC * 64 * 32 : 4096;
    constexpr int smem = NST * (BR + BC) * BKB + WR * WC * STRIP;      // operand ring + output strips
    static_assert(smem <= 160 * 1024, "LDS of one compute unit");
    auto kern = k_gemm_dma<WR, WC, TR, TC, BKB, EPI, HALVES, NST, LAY, MF>;
    static std::atomic<bool> lds_enabled[64];
    if (int e = enable_dynamic_lds(reinterpret_cast<const void*>(kern), smem, lds_enabled)) return e;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(WR * WC * 64), smem, st, da);
    return launch_status();
}

// MF: 16 = the 16x16 MFMAs (the large tile on products of several slabs), 32 = the 32x32 ones
// per_cu: workgroups a compute unit holds at once (their LDS and registers must allow it)
template <int WR, int WC, int TR, int TC, int BKB, int EPI, int NST, int LAY, int MF>
static int launch_dma(GemmArgs& a, int batch, hipStream_t st, int per_cu = 1) {
    constexpr int BR = WR * TR * 32, BC = WC * TC * 32;
    a.tiles_r = (int32_t)ceil_div(a.n, BR);
    a.tiles_c = (int32_t)ceil_div(a.m, BC);
    DmaArgs da;
    da.g = a;
    da.batch = batch;
    da.ntiles = a.tiles_r * a.tiles_c;
    const int64_t total = (int64_t)da.ntiles * batch;
    const int cus = compute_units() * per_cu;
    const int64_t grid = total < cus ? total : cus;
    // a last round of r <= grid/2 tiles is issued as 2r half tiles
    const int64_t r = total % grid;
    da.nfull = (uint32_t)total;
    da.nhalf = 0;
    if constexpr (TR % 2 == 0 && LAY == 0 && ((BR / 2 + BC) / (1024 / BKB)) % (WR * WC) == 0) {      // (a half tile's slab must split evenly over the waves too)
        if (r > 0 && 2 * r <= grid) {
            da.nfull = (uint32_t)(total - r);
            da.nhalf = (uint32_t)(2 * r);
            return launch_dma_kernel<WR, WC, TR, TC, BKB, EPI, true, NST, 0, MF>(da, (unsigned)grid, st);
        }
    }
    return launch_dma_kernel<WR, WC, TR, TC, BKB, EPI, false, NST, LAY, MF>(da, (unsigned)grid, st);
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
    if (out == nullptr || (k > 0 && any_null(A, B)) || (FUSED && any_null(srow, scol))) return CPMK_EBADARG;
    if (batch > 65535) {      // some kernels index the batch with the grid's z dimension: at most 65535 entries per call
        constexpr int64_t ESZ_OUT = FUSED ? 2 : 4;
        for (int64_t b0 = 0; b0 < batch; b0 += 65535) {
            const int32_t nb = (int32_t)(batch - b0 < 65535 ? batch - b0 : 65535);
            const int rc = gemm_dispatch<FUSED>(
                m, k, n, batchA == 1 ? 1 : nb, batchB == 1 ? 1 : nb, aT, bT,
                (const int8_t*)A + (batchA == 1 ? 0 : b0 * m * k), (const int8_t*)B + (batchB == 1 ? 0 : b0 * n * k),
                srow ? (const half_t*)srow + (bcr ? 0 : b0 * n) : nullptr, scol ? (const half_t*)scol + (bcc ? 0 : b0 * m) : nullptr,
                bcr, bcc, (int8_t*)out + b0 * n * m * ESZ_OUT, st);
            if (rc != 0) return rc;
        }
        return 0;
    }
    GemmArgs a;
    a.P = (const int8_t*)B; a.Q = (const int8_t*)A; a.out = out;
    a.srow = (const half_t*)srow; a.scol = (const half_t*)scol;
    a.strideP = batchB == 1 ? 0 : (int64_t)n * k;
    a.strideQ = batchA == 1 ? 0 : (int64_t)m * k;
    a.n = n; a.m = m; a.k = k; a.bc_row = bcr; a.bc_col = bcc;
    a.tiles_r = a.tiles_c = 0;
    a.edge_in = 0;
    // the tile kernel stores 16-byte pieces of output rows (8-byte halves where fp16 rows are not whole pieces: m % 8 == 4)
    const bool wide = aligned16(out);
    const bool p_kmajor = !bT, q_kmajor = aT != 0;
    const bool fast = p_kmajor && q_kmajor && k > 0 && (k % 16 == 0) && aligned16(A) && aligned16(B);
    if (fast && wide && (k % 64 == 0) && (int64_t)n * k < (1ll << 32) && (int64_t)m * k < (1ll << 32)) {
        // 256x256 tiles when they give most compute units a tile, else 128x128
        const int64_t big = ceil_div(n, 256) * ceil_div(m, 256) * batch;
        constexpr int EPI = FUSED ? kEpiDequant : kEpiInt32;
        if (k % 128 != 0) {
            // a depth of whole 64-byte but not whole 128-byte slabs (1600, 4544 ...): the same kernels on 64-byte slabs and
            // a ring of four stages -- twice the barriers per byte of K, 5-10 % behind the 128-byte form
            if (big * 4 >= compute_units() * 3 && n > 128 && m > 128) return launch_dma<2, 4, 4, 2, 64, EPI, 4, 0, 16>(a, batch, st);
            return launch_dma<2, 2, 2, 2, 64, EPI, kRingSmall, 0, 32>(a, batch, st);
        }
        // (a dimension of at most 128 would leave half or more of every 256-wide tile empty)
        if (big * 4 >= compute_units() * 3 && n > 128 && m > 128) return launch_dma<2, 4, 4, 2, 128, EPI, kRingBig, 0, 16>(a, batch, st);
        // 128x128 tiles, or 128x64 when even those leave a quarter of the compute units idle
        const int64_t mid = ceil_div(n, 128) * ceil_div(m, 128) * batch;
        // the smaller tiles finish a slab before a load from L2 returns: four ring stages keep them fed.  More
        // tiles than compute units but at most two each: a ring of two stages instead, which lets two
        // workgroups share a compute unit (2 x 80 KB of LDS) and all tiles run in one round, each
        // workgroup's waits covered by the other's MFMAs (6-11 % over 1.25-2 rounds of single workgroups)
        const int64_t cus = compute_units();
        if (mid * 4 >= cus * 3) {
            if (mid > cus && mid <= 2 * cus) return launch_dma<2, 2, 2, 2, 128, EPI, 2, 0, 32>(a, batch, st, 2);
            return launch_dma<2, 2, 2, 2, 128, EPI, kRingSmall, 0, 32>(a, batch, st);
        }
        const int64_t small = ceil_div(n, 128) * ceil_div(m, 64) * batch;
        if (small > cus && small <= 2 * cus) return launch_dma<2, 2, 2, 1, 128, EPI, 2, 0, 32>(a, batch, st, 2);
        return launch_dma<2, 2, 2, 1, 128, EPI, kRingSmall, 0, 32>(a, batch, st);
    }
    // a depth that is not whole 64-byte slabs (4000, 4048, 4100 ...): the tile kernels on 64-byte slabs, the rest of the
    // depth straight from memory into the fragments (k % 4 == 0 is the reference's precondition: rows of whole dwords)
    if (p_kmajor && q_kmajor && wide && k > 64 && (k % 4 == 0) && (reinterpret_cast<uintptr_t>(A) & 3u) == 0 &&
        (reinterpret_cast<uintptr_t>(B) & 3u) == 0 && (int64_t)n * k < (1ll << 32) && (int64_t)m * k < (1ll << 32)) {
        constexpr int EPI = FUSED ? kEpiDequant : kEpiInt32;
        const int64_t big = ceil_div(n, 256) * ceil_div(m, 256) * batch;
        const bool large = big * 4 >= compute_units() * 3 && n > 128 && m > 128;
        if (fast) return large ? launch_dma<2, 4, 4, 2, 64, EPI, 4, 4, 16>(a, batch, st) : launch_dma<2, 2, 2, 2, 64, EPI, kRingSmall, 4, 32>(a, batch, st);
        return large ? launch_dma<2, 4, 4, 2, 64, EPI, 4, 12, 16>(a, batch, st) : launch_dma<2, 2, 2, 2, 64, EPI, kRingSmall, 12, 32>(a, batch, st);
    }
    // an operand stored (K, rows): the tile kernel reads it as it lies and takes the fragments with transposing LDS reads
    // (rows of such an operand that are not whole 16-byte pieces: tiles that stay inside the matrix, which takes a matrix of
    // at least one tile)
    const bool in_p = !p_kmajor && n % 16 != 0, in_q = !q_kmajor && m % 16 != 0;
    if (!(p_kmajor && q_kmajor) && wide && k > 0 && (k % 128 == 0) && aligned16(A) && aligned16(B) && (!in_p || n >= 128) &&
        (!in_q || m >= 128) && (int64_t)n * k < (1ll << 32) && (int64_t)m * k < (1ll << 32)) {
        constexpr int EPI = FUSED ? kEpiDequant : kEpiInt32;
        // 256x256 tiles when they give most compute units a tile, else 128x128 (as for K-major operands)
        const int64_t big = ceil_div(n, 256) * ceil_div(m, 256) * batch;
        const bool large = big * 4 >= compute_units() * 3 && n > 128 && m > 128 && (!in_p || n >= 256) && (!in_q || m >= 256);
        a.edge_in = (in_p ? 1 : 0) | (in_q ? 2 : 0);
        switch ((p_kmajor ? 0 : 1) | (q_kmajor ? 0 : 2)) {
            case 1: return large ? launch_dma<2, 4, 4, 2, 128, EPI, 2, 1, 16>(a, batch, st) : launch_dma<2, 2, 2, 2, 128, EPI, kRingSmall, 1, 32>(a, batch, st);
            case 2: return large ? launch_dma<2, 4, 4, 2, 128, EPI, 2, 2, 16>(a, batch, st) : launch_dma<2, 2, 2, 2, 128, EPI, kRingSmall, 2, 32>(a, batch, st);
            default: return large ? launch_dma<2, 4, 4, 2, 128, EPI, 2, 3, 16>(a, batch, st) : launch_dma<2, 2, 2, 2, 128, EPI, kRingSmall, 3, 32>(a, batch, st);
        }
    }
    // one operand stored (K, rows) and a depth beyond one slab that is not whole slabs: the 32x32 form of the tile kernel,
    // the rest of the depth straight from memory into the fragments
    if (p_kmajor != q_kmajor && wide && k > 128 && (k % 4 == 0) && aligned16(A) && aligned16(B) && (!in_p || n >= 128) &&
        (!in_q || m >= 128) && (int64_t)n * k < (1ll << 32) && (int64_t)m * k < (1ll << 32)) {
        constexpr int EPI = FUSED ? kEpiDequant : kEpiInt32;
        a.edge_in = (in_p ? 1 : 0) | (in_q ? 2 : 0);
        if (!p_kmajor) return launch_dma<2, 2, 2, 2, 128, EPI, kRingSmall, 13, 32>(a, batch, st);
        return launch_dma<2, 2, 2, 2, 128, EPI, kRingSmall, 14, 32>(a, batch, st);
    }
    if (fast) {
        const int64_t t256 = ceil_div(n, 256) * ceil_div(m, 128) * batch;
        if (t256 >= 256) return launch_kmajor<2, 2, 4, 2, FUSED>(a, batch, st);
        return launch_kmajor<2, 2, 2, 2, FUSED>(a, batch, st);
    }
    // K-major rows that are only 4-byte aligned (k % 16 != 0; k % 4 == 0 always): the same kernel on 4-byte loads
    if (p_kmajor && q_kmajor && k > 0 && batch <= 65535 && (reinterpret_cast<uintptr_t>(A) & 3u) == 0 && (reinterpret_cast<uintptr_t>(B) & 3u) == 0 &&
        (FUSED ? (reinterpret_cast<uintptr_t>(out) & 1u) == 0 : (reinterpret_cast<uintptr_t>(out) & 3u) == 0)) {
        const int64_t t256 = ceil_div(n, 256) * ceil_div(m, 128) * batch;
        if (t256 >= 256) return launch_kmajor<2, 2, 4, 2, FUSED, true>(a, batch, st);
        return launch_kmajor<2, 2, 2, 2, FUSED, true>(a, batch, st);
    }
    // output rows are the grid's y dimension (65535 tiles of 64 rows): taller products go out in several launches
    for (int64_t r0 = 0; r0 < n; r0 += 65535ll * 64) {
        const int64_t nr = n - r0 < 65535ll * 64 ? n - r0 : 65535ll * 64;
        dim3 grid((unsigned)ceil_div(m, 64), (unsigned)ceil_div(nr, 64), (unsigned)batch);
        hipLaunchKernelGGL((k_gemm_generic<FUSED>), grid, dim3(256), 0, st, a, (int)p_kmajor, (int)q_kmajor, (int32_t)r0);
        if (int e = launch_status()) return e;
    }
    return 0;
}

// ---------------------------------------------------------------------------------------
// fp16 product (fp32 accumulation), any layout, size and alignment: 64x64 output tile, 64 halves of K per
// stage, four waves of one 32x32 MFMA tile each.  Shapes that are whole slabs and pieces run on the tile
// kernel above instead.
// ---------------------------------------------------------------------------------------
// V: halves per global access (4, 2 or 1: what the contiguous dimension of both operands and the alignment of the buffers allow).
template <int V>
__global__ __launch_bounds__(256) void k_gemm_f16_generic(GemmArgs a, int p_kmajor, int q_kmajor, int32_t row_base) {
    // Guarded loads bring a 64 x 64 piece of each operand into LDS with K contiguous (zeros past the edges,
    // so any size, layout and alignment works); each of the four waves then owns a 32 x 32 quarter of the tile and
    // multiplies with v_mfma_f32_32x32x16_f16.
    constexpr int T = 64, GK = 64, LD = GK + 4;        // rows of 136 bytes: 8-byte aligned fragment reads, spread over the banks
    __shared__ __attribute__((aligned(16))) half_t sP[T * LD];
    __shared__ __attribute__((aligned(16))) half_t sQ[T * LD];
    const int b = blockIdx.z;
    const int32_t k = a.k >> 1;                        // a.k is the row length in bytes
    const half_t* P = reinterpret_cast<const half_t*>(a.P + (int64_t)b * a.strideP);
    const half_t* Q = reinterpret_cast<const half_t*>(a.Q + (int64_t)b * a.strideQ);
    const int32_t j0 = row_base + blockIdx.y * T, i0 = blockIdx.x * T;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wr = wave >> 1, wc = wave & 1;
    const int lrow = lane & 31, lk = lane >> 5;
    float16_tv acc;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = 0.0f;
    typedef _Float16 halfV_t __attribute__((ext_vector_type(V > 1 ? V : 2)));
    // V halves of one operand's piece: along K for a K-major operand (one row), along the rows for one stored (K, rows).
    // A stage's pieces are requested one stage ahead into registers, so that their latency passes under the products.
    constexpr int S = T * GK / V / 256;       // accesses per thread, operand and stage
    auto place = [&](int kmajor, int q, int& r, int& kk) __attribute__((always_inline)) {
        if (kmajor) { r = q / (GK / V); kk = (q % (GK / V)) * V; } else { r = (q % (T / V)) * V; kk = q / (T / V); }
    };
    auto fetch = [&](half_t (&v)[V], const half_t* G, int kmajor, int32_t r0, int32_t L, int32_t k0, int q) __attribute__((always_inline)) {
        int r, kk;
        place(kmajor, q, r, kk);
        const int32_t row = r0 + r, kg = k0 + kk;
#pragma unroll
        for (int e = 0; e < V; ++e) v[e] = (half_t)0.0f;
        if (row < L && kg < k) {            // (L and k are multiples of V where the access runs along them)
            const half_t* src = kmajor ? G + ((int64_t)row * k + kg) : G + ((int64_t)kg * L + row);
            if constexpr (V > 1) {
                const halfV_t t = *reinterpret_cast<const halfV_t*>(src);
#pragma unroll
                for (int e = 0; e < V; ++e) v[e] = t[e];
            } else {
                v[0] = *src;
            }
        }
    };
    auto put = [&](half_t* sm, const half_t (&v)[V], int kmajor, int q) __attribute__((always_inline)) {
        int r, kk;
        place(kmajor, q, r, kk);
#pragma unroll
        for (int e = 0; e < V; ++e) sm[kmajor ? r * LD + kk + e : (r + e) * LD + kk] = v[e];
    };
    half_t rp[S][V], rq[S][V];
    auto fetch_all = [&](int32_t k0) __attribute__((always_inline)) {
#pragma unroll
        for (int s = 0; s < S; ++s) {
            fetch(rp[s], P, p_kmajor, j0, a.n, k0, tid + s * 256);
            fetch(rq[s], Q, q_kmajor, i0, a.m, k0, tid + s * 256);
        }
    };
    fetch_all(0);
    for (int32_t k0 = 0; k0 < k; k0 += GK) {
#pragma unroll
        for (int s = 0; s < S; ++s) {
            put(sP, rp[s], p_kmajor, tid + s * 256);
            put(sQ, rq[s], q_kmajor, tid + s * 256);
        }
        __syncthreads();
        if (k0 + GK < k) fetch_all(k0 + GK);
#pragma unroll
        for (int ks = 0; ks < GK / 16; ++ks) {
            // lane (lrow, lk): the 8 halves k = 16 ks + 8 lk .. + 7 of its row / column, as two 8-byte reads
            const half_t* pp = sP + (wr * 32 + lrow) * LD + ks * 16 + lk * 8;
            const half_t* qp = sQ + (wc * 32 + lrow) * LD + ks * 16 + lk * 8;
            const half4_t p0 = *reinterpret_cast<const half4_t*>(pp), p1 = *reinterpret_cast<const half4_t*>(pp + 4);
            const half4_t q0 = *reinterpret_cast<const half4_t*>(qp), q1 = *reinterpret_cast<const half4_t*>(qp + 4);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_shufflevector(p0, p1, 0, 1, 2, 3, 4, 5, 6, 7),
                                                         __builtin_shufflevector(q0, q1, 0, 1, 2, 3, 4, 5, 6, 7), acc, 0, 0, 0);
        }
        __syncthreads();
    }
    // accumulator register e of lane l: output row (e / 4) * 8 + (l / 32) * 4 + e % 4, column l % 32 of the wave's quarter
    const int64_t obase = (int64_t)b * a.n * a.m;
    const int32_t col = i0 + wc * 32 + lrow;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        const int32_t row = j0 + wr * 32 + (e >> 2) * 8 + lk * 4 + (e & 3);
        if (row < a.n && col < a.m) reinterpret_cast<half_t*>(a.out)[obase + (int64_t)row * a.m + col] = (half_t)acc[e];
    }
}

static int gemm_f16_dispatch(int32_t m, int32_t k, int32_t n, int32_t batchA, int32_t batchB, int aT, int bT,
                             const void* A, const void* B, void* out, hipStream_t st) {
    if (m < 0 || n < 0 || k < 0 || batchA < 1 || batchB < 1) return CPMK_EBADARG;
    if ((m % 2) || (n % 2) || (k % 2)) return CPMK_EALIGN;      // kernels/gemm.py:200
    if (!(batchA == batchB || batchA == 1 || batchB == 1)) return CPMK_EBADARG;   // :201
    const int batch = batchA > batchB ? batchA : batchB;
    if (m == 0 || n == 0) return 0;
    if (out == nullptr || (k > 0 && any_null(A, B))) return CPMK_EBADARG;
    if (k > (1 << 30)) return CPMK_ETOOBIG;
    if (batch > 65535) {      // (grid z: at most 65535 batch entries per call)
        for (int64_t b0 = 0; b0 < batch; b0 += 65535) {
            const int32_t nb = (int32_t)(batch - b0 < 65535 ? batch - b0 : 65535);
            const int rc = gemm_f16_dispatch(m, k, n, batchA == 1 ? 1 : nb, batchB == 1 ? 1 : nb, aT, bT,
                                             (const half_t*)A + (batchA == 1 ? 0 : b0 * m * k), (const half_t*)B + (batchB == 1 ? 0 : b0 * n * k),
                                             (half_t*)out + b0 * n * m, st);
            if (rc != 0) return rc;
        }
        return 0;
    }
    GemmArgs a;
    a.P = (const int8_t*)B; a.Q = (const int8_t*)A; a.out = out;
    a.srow = nullptr; a.scol = nullptr;
    a.strideP = batchB == 1 ? 0 : (int64_t)n * k * 2;          // bytes
    a.strideQ = batchA == 1 ? 0 : (int64_t)m * k * 2;
    a.n = n; a.m = m; a.k = k * 2; a.bc_row = 0; a.bc_col = 0;
    a.tiles_r = a.tiles_c = 0;
    a.edge_in = 0;
    const bool wide = aligned16(out) && m % 4 == 0;       // the tile kernel stores 16-byte pieces of output rows (8-byte halves where m % 8 == 4)
    const bool p_kmajor = !bT, q_kmajor = aT != 0;
    if (p_kmajor && q_kmajor && wide && k > 0 && (k % 32 == 0) && aligned16(A) && aligned16(B) &&
        (int64_t)n * k * 2 < (1ll << 32) && (int64_t)m * k * 2 < (1ll << 32)) {
        const int64_t big = ceil_div(n, 256) * ceil_div(m, 256) * batch;
        const bool whole128 = k % 64 == 0;       // the depth is whole 128-byte slabs (else whole 64-byte ones: 96, 160 ...)
        if (big * 4 >= compute_units() * 3 && n > 128 && m > 128) {
            if (whole128 && k >= 256) return launch_dma<2, 4, 4, 2, 128, kEpiF16, 2, 0, 16>(a, batch, st);
            // Products of a few slabs -- attention scores, K = 64 -- are all prologue and epilogue, bound by the stores (and
            // depths of whole 64-byte slabs only need this form anyway):
            // the 32x32 form is quicker there, and waves of 64 rows x 128 columns, whose row segments are 256 bytes,
            // store 5-15 % faster than waves of 128 x 64 (slabs of 64 bytes make room for their wider output strips)
            return launch_dma<4, 2, 2, 4, 64, kEpiF16, 2, 0, 32>(a, batch, st);
        }
        if (!whole128) return launch_dma<2, 2, 2, 2, 64, kEpiF16, kRingSmall, 0, 32>(a, batch, st);
        // (as for int8: more 128x128 tiles than compute units but at most two each -> two workgroups per compute unit)
        const int64_t mid = ceil_div(n, 128) * ceil_div(m, 128) * batch, cus = compute_units();
        if (mid > cus && mid <= 2 * cus) return launch_dma<2, 2, 2, 2, 128, kEpiF16, 2, 0, 32>(a, batch, st, 2);
        return launch_dma<2, 2, 2, 2, 128, kEpiF16, kRingSmall, 0, 32>(a, batch, st);
    }
    // a depth that is not whole 64-byte slabs (K = 40, 72, 500, 1000 ...): the same kernels, the rest of the depth straight
    // from memory into the fragments
    if (p_kmajor && q_kmajor && wide && k > 32 && (reinterpret_cast<uintptr_t>(A) & 3u) == 0 && (reinterpret_cast<uintptr_t>(B) & 3u) == 0 &&
        (int64_t)n * k * 2 < (1ll << 32) && (int64_t)m * k * 2 < (1ll << 32)) {
        const int64_t big = ceil_div(n, 256) * ceil_div(m, 256) * batch;
        const bool large = big * 4 >= compute_units() * 3 && n > 128 && m > 128;
        if (k % 8 == 0 && aligned16(A) && aligned16(B))       // whole, aligned 16-byte pieces
            return large ? launch_dma<4, 2, 2, 4, 64, kEpiF16, 2, 4, 32>(a, batch, st) : launch_dma<2, 2, 2, 2, 64, kEpiF16, kRingSmall, 4, 32>(a, batch, st);
        return large ? launch_dma<4, 2, 2, 4, 64, kEpiF16, 2, 12, 32>(a, batch, st) : launch_dma<2, 2, 2, 2, 64, kEpiF16, kRingSmall, 12, 32>(a, batch, st);
    }
    // an operand stored (K, rows): the tile kernel reads it as it lies, with transposing LDS reads for the fragments
    // (rows of such an operand that are not whole 16-byte pieces, but whole 8-byte ones: tiles that stay inside the matrix,
    // which takes a matrix of at least one tile)
    const bool in_p = !p_kmajor && n % 8 != 0, in_q = !q_kmajor && m % 8 != 0;
    const bool low = n <= 64;                // 64 x 256 tiles for few output rows (attention: probabilities x values)
    if (!(p_kmajor && q_kmajor) && wide && k > 0 && (k % 64 == 0) && aligned16(A) && aligned16(B) &&
        (!in_p || (n % 4 == 0 && n >= 128)) && (!in_q || (m % 4 == 0 && m >= (low ? 256 : 128))) &&
        (int64_t)n * k * 2 < (1ll << 32) && (int64_t)m * k * 2 < (1ll << 32)) {
        const int lay = (p_kmajor ? 0 : 1) | (q_kmajor ? 0 : 2);
        // else 256x256 tiles when they give most compute units a tile, else 128x128 (as for K-major operands)
        const int64_t big = ceil_div(n, 256) * ceil_div(m, 256) * batch;
        const bool large = big * 4 >= compute_units() * 3 && n > 128 && m > 128 && (!in_p || n >= 256) && (!in_q || m >= 256);
        a.edge_in = (in_p ? 1 : 0) | (in_q ? 2 : 0);
        switch (lay) {
            case 1:
                if (low) return launch_dma<1, 4, 2, 2, 128, kEpiF16, 3, 1, 32>(a, batch, st);
                return large ? launch_dma<2, 4, 4, 2, 128, kEpiF16, 2, 1, 16>(a, batch, st) : launch_dma<2, 2, 2, 2, 128, kEpiF16, kRingSmall, 1, 32>(a, batch, st);
            case 2:
                if (low) return launch_dma<1, 4, 2, 2, 128, kEpiF16, 3, 2, 32>(a, batch, st);
                return large ? launch_dma<2, 4, 4, 2, 128, kEpiF16, 2, 2, 16>(a, batch, st) : launch_dma<2, 2, 2, 2, 128, kEpiF16, kRingSmall, 2, 32>(a, batch, st);
            default:
                if (low) return launch_dma<1, 4, 2, 2, 128, kEpiF16, 3, 3, 32>(a, batch, st);
                return large ? launch_dma<2, 4, 4, 2, 128, kEpiF16, 2, 3, 16>(a, batch, st) : launch_dma<2, 2, 2, 2, 128, kEpiF16, kRingSmall, 3, 32>(a, batch, st);
        }
    }
    // one operand stored (K, rows) and a depth that is not whole slabs (attention: probabilities x values over 500 keys):
    // the 32x32 form of the tile kernel, the rest of the depth straight from memory into the fragments
    if (p_kmajor != q_kmajor && wide && k > 64 && (k % 64 != 0) && aligned16(A) && aligned16(B) &&
        (!in_p || (n % 4 == 0 && n >= 128)) && (!in_q || (m % 4 == 0 && m >= (low ? 256 : 128))) &&
        (int64_t)n * k * 2 < (1ll << 32) && (int64_t)m * k * 2 < (1ll << 32)) {
        a.edge_in = (in_p ? 1 : 0) | (in_q ? 2 : 0);
        if (!p_kmajor) return low ? launch_dma<1, 4, 2, 2, 128, kEpiF16, 3, 13, 32>(a, batch, st) : launch_dma<2, 2, 2, 2, 128, kEpiF16, kRingSmall, 13, 32>(a, batch, st);
        return low ? launch_dma<1, 4, 2, 2, 128, kEpiF16, 3, 14, 32>(a, batch, st) : launch_dma<2, 2, 2, 2, 128, kEpiF16, kRingSmall, 14, 32>(a, batch, st);
    }
    for (int64_t r0 = 0; r0 < n; r0 += 65535ll * 64) {        // (rows beyond the grid's y dimension: several launches)
        const int64_t nr = n - r0 < 65535ll * 64 ? n - r0 : 65535ll * 64;
        dim3 grid((unsigned)ceil_div(m, 64), (unsigned)ceil_div(nr, 64), (unsigned)batch);
        // the widest access both operands allow: their contiguous dimension a multiple of it, their buffers aligned to it
        const int32_t cp = p_kmajor ? k : n, cq = q_kmajor ? k : m;
        const uintptr_t al = reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B);
        if (cp % 4 == 0 && cq % 4 == 0 && (al & 7u) == 0)
            hipLaunchKernelGGL(k_gemm_f16_generic<4>, grid, dim3(256), 0, st, a, (int)p_kmajor, (int)q_kmajor, (int32_t)r0);
        else if (cp % 2 == 0 && cq % 2 == 0 && (al & 3u) == 0)
            hipLaunchKernelGGL(k_gemm_f16_generic<2>, grid, dim3(256), 0, st, a, (int)p_kmajor, (int)q_kmajor, (int32_t)r0);
        else
            hipLaunchKernelGGL(k_gemm_f16_generic<1>, grid, dim3(256), 0, st, a, (int)p_kmajor, (int)q_kmajor, (int32_t)r0);
        if (int e = launch_status()) return e;
    }
    return 0;
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

int cpmk_gemm_fp16(int32_t m, int32_t k, int32_t n, int32_t batchA, int32_t batchB, int aT, int bT,
                   const void* A, const void* B, void* out, void* stream) {
    clear_stale_error();
    return gemm_f16_dispatch(m, k, n, batchA, batchB, aT, bT, A, B, out, (hipStream_t)stream);
}

}  // extern "C"
