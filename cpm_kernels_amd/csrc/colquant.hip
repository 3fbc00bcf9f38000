// Per-column absmax scales and rounding of a (batch, n, m) fp16 tensor in one pass over HBM:
//   scale[b, j] = fp16(max_i |mat[b,i,j]| / 127),   q = int8(rint(mat[b,i,j] / scale[b,j]))
// i.e. cu_gemm_calc_scale_transpose followed by cu_gemm_round_transpose (cuda/gemm.cu:22-33,
// 79-98), with q written either in place (b, n, m) or transposed (b, m, n).  The transposed form
// is what lets torch-level bmm feed operands given as (batch, K, N) to the K-major int8 GEMM
// (the reference's GEMMInt8.forward, torch/gemm.py:84-113, quantises such an operand along
// dim 1 and leaves the transposition to cuBLASLt).
#include "dim1.h"
#include "exchange.h"

namespace cpmk {

// 64 columns x 512 rows per workgroup; taller columns are shared by a team (exchange.h) that
// exchanges the per-column maxima.  Lane (cg = tid % 8, rg = tid / 8) holds 8 columns of the 8
// consecutive rows rg*8 .. rg*8+7, so that its int8 results are 8 contiguous bytes in either
// output layout.
// (two 512-thread workgroups share a compute unit: at most 128 registers per lane)
// NTH: the tile's 128-byte row segments are whole cache lines (m % 64 == 0, the matrix on a 128-byte boundary): the input is
// read with the non-temporal hint.  Elsewhere a line is shared with the neighbouring tile and has to stay in L2 for it.
// UA: any m and alignment: a piece inside its row still moves whole, at whatever address it lies (global accesses need
// no alignment); the piece across a row's end is read (and its scales and, not transposed, its int8 values are
// written) in at most three narrower accesses.
template <int NT, bool TRANSPOSED, bool NTH, bool UA = false>
__global__ __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(4, 4))) void k_col_quantize_team(int32_t n, int32_t m, int32_t tiles_per_batch, int32_t parts,
                                                          const half_t* __restrict__ mat, half_t* __restrict__ scale,
                                                          int8_t* __restrict__ out, uint32_t nteams, XchLaunch xl) {
    constexpr int LPR = 8, R = 8, COLS = 64, ROWS = NT / LPR * R;
    uint64_t* const xch = xl.region;
    const uint32_t tag = xl.tag;
    __shared__ float lds[(NT / 64 + 1) * COLS];
    __shared__ float tot[COLS];
    __shared__ __attribute__((aligned(16))) int8_t tbuf[TRANSPOSED ? COLS * ROWS : 16];       // the transposed int8 tile on its way out
    const int tid = threadIdx.x, cg = tid % LPR, rg = tid / LPR;
    XchMember me;
    if (!xch_member(blockIdx.x, parts, nteams, me)) return;
    const uint32_t part = me.part, team = me.team;
    const uint32_t b = team / tiles_per_batch, ct = team - b * tiles_per_batch;
    const int32_t col0 = ct * COLS + cg * 8;
    const int32_t row0 = part * ROWS + rg * 8;           // this lane's first row
    const int64_t boff = (int64_t)b * n * m;

    half8_t v[R];
#pragma unroll
    for (int p = 0; p < R; ++p) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[p][e] = (half_t)0.0f;
        if constexpr (UA) {
            if (row0 + p < n) {
                const half_t* src = mat + boff + ((uint32_t)(row0 + p) * (uint32_t)m + (uint32_t)col0);
                if (col0 + 8 <= m) {
                    v[p] = load_half8_any(src);
                } else if (col0 < m) {
                    v[p] = load_half8_head_any(src, m & 7, v[p]);
                }
            }
        } else if (row0 + p < n && col0 < m) {
            const half8_t* src = reinterpret_cast<const half8_t*>(mat + boff + ((uint32_t)(row0 + p) * (uint32_t)m + (uint32_t)col0));
            v[p] = NTH ? __builtin_nontemporal_load(src) : *src;        // read once; the int8 output below is what the next kernel wants in cache
        }
    }
    // |x| maxima of the lane's 8 columns as integers; a NaN among them (rare) repeats the maximum in
    // floating point, which skips NaN elements
    ushort8_t um = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int p = 0; p < R; ++p) um = absbits_max(um, v[p]);
    half8_t hm = __builtin_bit_cast(half8_t, um);
    if (absbits_max_of(um) > 0x7c00u) {
        hm = __builtin_elementwise_abs(v[0]);
#pragma unroll
        for (int p = 1; p < R; ++p) hm = __builtin_elementwise_max(hm, __builtin_elementwise_abs(v[p]));
    }
    float mx[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) mx[e] = (float)hm[e];
    if (parts == 1) {
        coltile_reduce<NT, LPR, 1, true>(mx, lds);       // every lane: the maxima of its 8 columns
    } else {
        uint64_t* team_slots = xch + (size_t)team * parts * kXchVals;
        // this part's maxima go straight from the reduction to its slot
        coltile_reduce_to<NT, LPR, 1, true>(mx, lds, [&](int i, float r) { xch_post(team_slots + (size_t)part * kXchVals, i, r, tag); });
        if (tid < COLS) {
            const uint64_t deadline = wall_clock64() + kXchTimeoutTicks;
            float M = 0.0f;
            bool ok = true;
            for (int32_t q0 = 0; q0 < parts; q0 += 8) {
                float x[8];
                ok &= xch_gather<8>(team_slots, parts, q0, tid, tag, deadline, x);
#pragma unroll
                for (int j = 0; j < 8; ++j) M = fmaxf(M, x[j]);       // maxima are >= 0: absent parts (zeros) do not matter
            }
            tot[tid] = ok ? M : __builtin_nanf("");
            if (!ok) xch_flag(xl, kXchStatusTimeout);
        }
        __syncthreads();
#pragma unroll
        for (int e = 0; e < 8; ++e) mx[e] = tot[cg * 8 + e];
    }

    half8_t sh;
    float s[8], y[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        sh[e] = scale_from_absmax(mx[e]);
        s[e] = (float)sh[e];
        y[e] = 1.0f / s[e];
    }
    if (part == 0 && rg == 0) {
        if constexpr (UA) {
            if (col0 + 8 <= m) {
                store_half8_any(scale + (int64_t)b * m + col0, sh);
            } else if (col0 < m) {
                store_half8_head_any(scale + (int64_t)b * m + col0, m & 7, sh);
            }
        } else if (col0 < m) {
            *reinterpret_cast<half8_t*>(scale + (int64_t)b * m + col0) = sh;
        }
    }

    uint32_t q[R][2];       // [row p][columns 0-3 | 4-7], one byte each
    bool normal = true;
#pragma unroll
    for (int e = 0; e < 8; ++e) normal = normal && scale_is_normal(sh[e]);
    if (__builtin_amdgcn_ballot_w64(!normal) == 0) {    // every scale of the wave's columns is a normal number: the short rounding sequence
#pragma unroll
        for (int p = 0; p < R; ++p) {
            uint32_t t[8];
            int4_t vp = __builtin_bit_cast(int4_t, v[p]);
            asm volatile("" : "+v"(vp));             // keeps the fp32 conversions of the two paths apart (hoisted above the branch they hold 64 registers)
            const half8_t vh = __builtin_bit_cast(half8_t, vp);
#pragma unroll
            for (int e = 0; e < 8; ++e) t[e] = quant_i8_own_scale_bits((float)vh[e], s[e], y[e]);
            q[p][0] = pack4_i8((int32_t)t[0], (int32_t)t[1], (int32_t)t[2], (int32_t)t[3]);
            q[p][1] = pack4_i8((int32_t)t[4], (int32_t)t[5], (int32_t)t[6], (int32_t)t[7]);
            __builtin_amdgcn_sched_barrier(0);      // one row at a time: interleaving all 64 elements costs registers
        }
    } else {
#pragma unroll
        for (int p = 0; p < R; ++p) {
            int32_t t[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) t[e] = quant_i8_rcp((float)v[p][e], s[e], y[e]);
            q[p][0] = pack4_i8(t[0], t[1], t[2], t[3]);
            q[p][1] = pack4_i8(t[4], t[5], t[6], t[7]);
        }
    }
    if (col0 < m) {
        if constexpr (!TRANSPOSED) {
#pragma unroll
            for (int p = 0; p < R; ++p)
                if (row0 + p < n) {
                    int8_t* dst = out + boff + ((uint32_t)(row0 + p) * (uint32_t)m + (uint32_t)col0);
                    if constexpr (UA) {
                        if (col0 + 8 <= m) {
                            store_byte8_any(dst, q[p][0], q[p][1]);
                        } else {
                            store_byte8_head_any(dst, m & 7, q[p][0], q[p][1]);
                        }
                    } else {
                        *reinterpret_cast<uint2_t*>(dst) = uint2_t{q[p][0], q[p][1]};
                    }
                }
        }
    }
    if constexpr (TRANSPOSED) {
        // The tile leaves through LDS as 64 columns x ROWS bytes: a lane's 8 rows of a column are 8
        // bytes there, and 32 lanes then store one column's ROWS bytes as one contiguous run (16 bytes
        // per lane) instead of eight lanes storing 64 bytes of it.  8-byte slot s of column c sits at
        // slot s ^ ((c / 8) * 8): the 64 lanes of a writing wave cover every bank equally, and the
        // 16-byte reads stay pairs of neighbouring slots.
        static_assert(ROWS == 512, "one column of the tile is 64 slots of 8 bytes");
        // 4x4 byte transposes with v_perm_b32 (selector bytes 0-3 pick from the second operand, 4-7 from
        // the first): tr[h][e4][k] = rows 4k .. 4k+3 of column 4h + e4
        uint32_t tr[2][4][2];
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int k = 0; k < 2; ++k) {
                const uint32_t r0 = q[4 * k][h], r1 = q[4 * k + 1][h], r2 = q[4 * k + 2][h], r3 = q[4 * k + 3][h];
                const uint32_t a01 = __builtin_amdgcn_perm(r1, r0, 0x05010400u), b01 = __builtin_amdgcn_perm(r1, r0, 0x07030602u);
                const uint32_t a23 = __builtin_amdgcn_perm(r3, r2, 0x05010400u), b23 = __builtin_amdgcn_perm(r3, r2, 0x07030602u);
                tr[h][0][k] = __builtin_amdgcn_perm(a23, a01, 0x05040100u);
                tr[h][1][k] = __builtin_amdgcn_perm(a23, a01, 0x07060302u);
                tr[h][2][k] = __builtin_amdgcn_perm(b23, b01, 0x05040100u);
                tr[h][3][k] = __builtin_amdgcn_perm(b23, b01, 0x07060302u);
            }
#pragma unroll
        for (int e = 0; e < 8; ++e)
            *reinterpret_cast<uint2_t*>(tbuf + (cg * 8 + e) * ROWS + ((rg ^ (cg << 3)) << 3)) = uint2_t{tr[e >> 2][e & 3][0], tr[e >> 2][e & 3][1]};
        __syncthreads();
        const int piece = tid & 31;                                  // 16 rows of a column
        const int32_t prow = part * ROWS + piece * 16;
#pragma unroll
        for (int ps = 0; ps < COLS / (NT / 32); ++ps) {
            const int c = ps * (NT / 32) + (tid >> 5);
            const int32_t col = ct * COLS + c;
            const int4_t w = *reinterpret_cast<const int4_t*>(tbuf + c * ROWS + (((piece * 2) ^ ((c >> 3) << 3)) << 3));
            int8_t* dst = out + boff + ((uint32_t)col * (uint32_t)n + (uint32_t)prow);
            if (col < m) {             // n % 8 == 0: a piece is whole, half or not there
                if (prow + 16 <= n) *reinterpret_cast<int4_t*>(dst) = w;
                else if (prow + 8 <= n) *reinterpret_cast<uint2_t*>(dst) = uint2_t{(uint32_t)w.x, (uint32_t)w.y};
            }
        }
    }
    if (parts > 1 && tid < 64) xch_retire(xl, team, parts);
}

// Any shape: rounding with per-column scales into the transposed layout, one element per thread.
__global__ __launch_bounds__(256) void k_round_cols_transposed(int64_t total, int32_t n, int32_t m,
                                                               const half_t* __restrict__ mat,
                                                               const half_t* __restrict__ scale,
                                                               int8_t* __restrict__ out) {
    const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (gid >= total) return;
    const int64_t bi = gid / m;                 // b*n + i
    const int32_t j = (int32_t)(gid - bi * m);
    const int64_t b = bi / n;
    const int32_t i = (int32_t)(bi - b * n);
    out[(b * m + j) * n + i] = (int8_t)quant_i8((float)mat[gid], (float)scale[b * m + j]);
}

}  // namespace cpmk

using namespace cpmk;

extern "C" {

int cpmk_gemm_calc_scale_transpose(int32_t, int32_t, int32_t, const void*, void*, void*);
int cpmk_gemm_round_transpose(int32_t, int32_t, int32_t, const void*, const void*, void*, void*);

int cpmk_gemm_quantize_cols(int32_t batch, int32_t n, int32_t m, const void* mat, void* scale, void* out,
                            int out_transposed, void* stream) {
    clear_stale_error();
    if (batch < 0 || n < 0 || m < 0) return CPMK_EBADARG;
    if ((int64_t)batch * m == 0) return 0;
    if (n == 0) return cpmk_gemm_calc_scale_transpose(batch, n, m, mat, scale, stream);       // (columns of no elements: scale 0, nothing to round)
    if (any_null(mat, scale, out)) return CPMK_EBADARG;
    hipStream_t st = (hipStream_t)stream;
    // a team here only exchanges one maximum per column and gathers it in a loop over the parts, so
    // it may be larger than the teams of the kernels that keep per-part values in registers
    // (16384 rows; far fewer workgroups than are resident at once, which is what progress needs)
    constexpr int64_t kColMaxParts = 32;
    const int64_t tiles = ceil_div(m, 64), parts = ceil_div(n, 512);
    // rows of whole 16-byte pieces in aligned buffers: 16-byte accesses; any other width or alignment: the same kernel moving
    // its columns one by one (the transposed output runs along n either way)
    const bool wide = (m % 8 == 0) && aligned16(mat) && aligned16(scale) && ((reinterpret_cast<uintptr_t>(out) & 7u) == 0);
    const bool team_ok = (!out_transposed || (n % 8 == 0 && (reinterpret_cast<uintptr_t>(out) & 7u) == 0)) && (int64_t)n * m < (1ll << 31) &&
                         parts <= kColMaxParts && tiles * parts <= kXchSlots;
    if (team_ok) {
        // teams use one packet slot per (team, part): batches beyond the pool go out in several launches
        const int64_t per_launch = parts > 1 ? kXchSlots / (tiles * parts) : ((1ll << 31) - 8) / (tiles * parts);
        bool no_slots = false;
        for (int64_t b0 = 0; b0 < batch; b0 += per_launch) {
            const int64_t nb = batch - b0 < per_launch ? batch - b0 : per_launch;
            XchScope xs;
            if (parts > 1) {
                const int rc = xs.begin(tiles * nb * parts, st);
                if (rc == kXchFull && b0 == 0) {
                    no_slots = true;       // recorded into a graph and the capture reserve is used up: the separate kernels below
                    break;
                }
                if (rc != 0) return rc == kXchFull ? CPMK_ETOOBIG : rc;
            }
            const bool lines = m % 64 == 0 && (reinterpret_cast<uintptr_t>(mat) & 127u) == 0;
            auto go = [&](auto kern) {
                hipLaunchKernelGGL(kern, dim3((unsigned)xch_team_grid(tiles * nb, parts)), dim3(512), 0, st, n, m, (int32_t)tiles, (int32_t)parts,
                                   (const half_t*)mat + b0 * n * m, (half_t*)scale + b0 * m, (int8_t*)out + b0 * n * m, (uint32_t)(tiles * nb), xs.xl);
            };
            if (out_transposed) {
                if (!wide) go(k_col_quantize_team<512, true, false, true>);
                else if (lines) go(k_col_quantize_team<512, true, true>);
                else go(k_col_quantize_team<512, true, false>);
            } else {
                if (!wide) go(k_col_quantize_team<512, false, false, true>);
                else if (lines) go(k_col_quantize_team<512, false, true>);
                else go(k_col_quantize_team<512, false, false>);
            }
            const int e = launch_status();
            const int rc2 = xs.end();
            if (e != 0 || rc2 != 0) return e ? e : rc2;
        }
        if (!no_slots) return 0;
    }
    if (int e = cpmk_gemm_calc_scale_transpose(batch, n, m, mat, scale, stream)) return e;
    if (!out_transposed) return cpmk_gemm_round_transpose(batch, n, m, mat, scale, out, stream);
    const int64_t total = (int64_t)batch * n * m;
    hipLaunchKernelGGL(k_round_cols_transposed, dim3((unsigned)ceil_div(total, 256)), dim3(256), 0, st, total, n, m,
                       (const half_t*)mat, (const half_t*)scale, (int8_t*)out);
    return launch_status();
}

}  // extern "C"
