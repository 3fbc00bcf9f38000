// Normalisation over dim 1 of (batch, n, m) fp16 and over contiguous rows (decode step):
//   mean = rd_mean ? sum x / n : 0;  var = sum x^2 / n - mean^2;
//   y = fp16( (x - mean) * rsqrt(var + eps) )            (cuda/layernorm.cu:6-71, :343-381)
// optionally followed, on the fp16-rounded y, by the affine of cu_arith_ln_mul_add /
// cu_arith_ln_mul (cuda/arith.cu:97-127): fp16 fma(y, alpha[i], beta[i]) or y * alpha[i].
#include "dim1.h"
#include "exchange.h"
#include <mutex>


namespace cpmk {

// One row's coefficients applied to the lane's 8 columns with packed fp16 operations (a singly rounded
// fma, or a product): two elements per instruction, and `has_beta`, which is the same for the whole
// launch, decides between two instruction streams instead of between two results per element.
__device__ inline half8_t affine8(half8_t y, half_t a, half_t b, bool has_beta) {
    const half8_t a8 = {a, a, a, a, a, a, a, a};
    if (has_beta) {
        const half8_t b8 = {b, b, b, b, b, b, b, b};
        return __builtin_elementwise_fma(y, a8, b8);
    }
    return y * a8;
}

// Single pass: the whole (n x LPR*8) column tile lives in registers.  Tiles of whole cache lines (LPR == 8) are
// read and written with the non-temporal hint: every byte is touched once (8 x 4096 x 512 through the team
// kernel: 17.2 -> 15.2 us).
// MODE 0: 16-byte accesses, non-temporal where a tile's row segments are whole cache lines; 1: 16-byte accesses without
// the hint (rows that do not start on 128-byte boundaries); 2: any m and alignment, element by element (dim1.h).
template <int NT, int LPR, int R, bool AFF, int MODE = 0>
__global__ __launch_bounds__(NT) void k_layernorm_tile(int32_t n, int32_t m, int32_t tiles_per_batch,
                                                       const half_t* mat, half_t* out,
                                                       const half_t* __restrict__ alpha,
                                                       const half_t* __restrict__ beta, float eps,
                                                       int rd_mean) {
    using T = ColTile<NT, LPR, R>;
    __shared__ float lds[(T::NW + 1) * T::COLS * 2];
    __shared__ half_t coef[2][T::ROWS];   // alpha and beta of the tile's rows
    const uint32_t t = xcd_remap(blockIdx.x, gridDim.x);
    const uint32_t b = t / tiles_per_batch, ct = t - b * tiles_per_batch;
    const int32_t col0 = ct * T::COLS + (threadIdx.x % LPR) * 8;
    const int64_t boff = (int64_t)b * n * m;

    // the affine coefficients of the tile's rows, contiguous loads requested ahead of the tile (loads
    // return in order: behind the tile they would hold the sums below back until its last piece had
    // arrived) and parked in LDS until the output pass (the barriers of the reduction order write and reads)
    constexpr int CPT = (T::ROWS + NT - 1) / NT;       // coefficient pairs per thread
    half_t ca[CPT], cb[CPT];
    if constexpr (AFF) {
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const int32_t row = min((int32_t)(threadIdx.x + i * NT), n - 1);
            ca[i] = alpha[row];
            cb[i] = beta != nullptr ? beta[row] : (half_t)0.0f;
        }
    }
    half8_t v[R];
    coltile_load<NT, LPR, R, LPR == 8 && MODE == 0, MODE == 2>(v, mat + boff, n, m, col0, (half_t)0.0f);
    if constexpr (AFF) {
#pragma unroll
        for (int i = 0; i < CPT; ++i) {
            const int r = threadIdx.x + i * NT;
            if (r < T::ROWS) {
                coef[0][r] = ca[i];
                coef[1][r] = cb[i];
            }
        }
    }

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
        if constexpr (AFF) y = affine8(y, coef[0][p * T::RPP + rg], coef[1][p * T::RPP + rg], beta != nullptr);
        v[p] = y;
    }
    coltile_store<NT, LPR, R, LPR == 8 && MODE == 0, MODE == 2>(v, out + boff, n, m, col0);
}

// Tall columns.  A register tile holds T::ROWS rows of 64 columns (128-byte row segments, whole
// cache lines); narrower tiles would hold more rows but touch only part of every line.  The n
// rows of a 64-column tile are therefore split over a team of `parts` workgroups (exchange.h):
// each keeps its own rows in registers, posts its partial column sums, adds up the team's
// partials in part order (so the result does not depend on timing) and normalises its rows.
// A workgroup reads and writes only its own rows: out may alias mat.
template <int NT, int R, bool AFF, int MODE = 0>
__global__ __launch_bounds__(NT) void k_layernorm_team(int32_t n, int32_t m, int32_t tiles_per_batch, int32_t parts,
                                                       const half_t* mat, half_t* out,
                                                       const half_t* __restrict__ alpha,
                                                       const half_t* __restrict__ beta, float eps, int rd_mean,
                                                       uint32_t nteams, XchLaunch xl) {
    constexpr int LPR = 8;
    using T = ColTile<NT, LPR, R>;
    static_assert(T::COLS * 2 == kXchVals, "slot layout");
    uint64_t* const xch = xl.region;
    const uint32_t tag = xl.tag;
    __shared__ float lds[(T::NW + 1) * T::COLS * 2];
    __shared__ float tot[kXchVals];
    __shared__ half_t coef[2][NT];        // alpha and beta of this workgroup's rows (T::ROWS == NT)
    static_assert(T::ROWS == NT, "one affine coefficient pair per thread");
    const int tid = threadIdx.x;
    XchMember me;
    if (!xch_member(blockIdx.x, parts, nteams, me)) return;
    const uint32_t part = me.part, team = me.team;
    const uint32_t b = team / tiles_per_batch, ct = team - b * tiles_per_batch;
    const int32_t col0 = ct * T::COLS + (tid % LPR) * 8;
    const int32_t own0 = part * T::ROWS;                 // first row this workgroup normalises
    const int32_t own_n = min(T::ROWS, n - own0);        // > 0 by construction
    const int64_t boff = (int64_t)b * n * m + (int64_t)own0 * m;

    // The affine coefficients of the workgroup's rows: one pair per thread, contiguous, parked in
    // LDS until the output pass (a thread's own rows are RPP apart; fetching them lane by lane
    // took 2 x R two-byte loads per thread, as many load instructions again as the tile itself).
    // Requested ahead of the tile: loads return in order, so behind the tile they would hold the
    // sums below back until the last piece of the tile had arrived.
    const int rg = tid / LPR;
    half_t ca = (half_t)0.0f, cb = (half_t)0.0f;
    if constexpr (AFF) {
        const int32_t row = min(own0 + tid, n - 1);
        ca = alpha[row];
        if (beta != nullptr) cb = beta[row];
    }
    half8_t v[R];
    coltile_load<NT, LPR, R, MODE == 0, MODE == 2>(v, mat + boff, own_n, m, col0, (half_t)0.0f);
    if constexpr (AFF) {
        coef[0][tid] = ca;
        coef[1][tid] = cb;
    }
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
    // packet g*64 + c of a slot: statistic g (0 sum, 1 sum of squares) of tile column c; the part's own
    // totals go straight from the reduction to its slot
    uint64_t* team_slots = xch + (size_t)team * parts * kXchVals;
    coltile_reduce_to<NT, LPR, 2, false>(s, lds, [&](int i, float r) { xch_post(team_slots + (size_t)part * kXchVals, i, r, tag); });
    // One thread per column collects the team's sums of that column, both statistics, and turns them into
    // the column's mean and reciprocal deviation once; the 128 lanes that hold rows of the column then read
    // the two numbers instead of each repeating the two divisions and the square root.
    if (tid < T::COLS) {
        const uint64_t deadline = wall_clock64() + kXchTimeoutTicks;
        float sum = 0.0f, sq = 0.0f;
        bool ok = true;
        for (int32_t q0 = 0; q0 < parts; q0 += 4) {
            float x[4], y[4];
            ok &= xch_gather2<4>(team_slots, parts, q0, tid, T::COLS + tid, tag, deadline, x, y);      // both statistics of four parts in one round trip
#pragma unroll
            for (int j = 0; j < 4; ++j) {                  // in part order; absent parts are zeros
                sum += x[j];
                sq += y[j];
            }
        }
        const float fn = (float)n;
        float var = sq / fn, mu = 0.0f;
        if (rd_mean) {
            mu = sum / fn;
            var -= mu * mu;
        }
        tot[tid] = mu;
        tot[T::COLS + tid] = ok ? rsqrtf(var + eps) : __builtin_nanf("");
        if (!ok) xch_flag(xl, kXchStatusTimeout);
    }
    __syncthreads();
    const int cg = tid % LPR;
    float mean[8], rstd[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        mean[e] = tot[cg * 8 + e];
        rstd[e] = tot[T::COLS + cg * 8 + e];
    }
#pragma unroll
    for (int p = 0; p < R; ++p) {
        half8_t y;
#pragma unroll
        for (int e = 0; e < 8; ++e) y[e] = round_f16(((float)v[p][e] - mean[e]) * rstd[e]);
        if constexpr (AFF) y = affine8(y, coef[0][p * T::RPP + rg], coef[1][p * T::RPP + rg], beta != nullptr);
        v[p] = y;
    }
    coltile_store<NT, LPR, R, MODE == 0, MODE == 2>(v, out + boff, own_n, m, col0);
    if (tid < 64) xch_retire(xl, team, parts);     // after the barrier above: this workgroup holds all it needs
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

template <int LPR, int R, int MODE = 0>
static void launch_tile(int32_t batch, int32_t n, int32_t m, const half_t* mat, half_t* out, const half_t* alpha,
                        const half_t* beta, float eps, int rd_mean, hipStream_t st) {
    constexpr int NT = 1024;
    const int32_t tiles = (int32_t)ceil_div(m, LPR * 8);
    if (alpha != nullptr)
        hipLaunchKernelGGL((k_layernorm_tile<NT, LPR, R, true, MODE>), dim3((unsigned)((int64_t)tiles * batch)), dim3(NT), 0, st, n,
                           m, tiles, mat, out, alpha, beta, eps, rd_mean);
    else
        hipLaunchKernelGGL((k_layernorm_tile<NT, LPR, R, false, MODE>), dim3((unsigned)((int64_t)tiles * batch)), dim3(NT), 0, st, n,
                           m, tiles, mat, out, alpha, beta, eps, rd_mean);
}

template <int LPR, int MODE = 0>
static bool launch_tile_r(int r, int32_t batch, int32_t n, int32_t m, const half_t* mat, half_t* out,
                          const half_t* alpha, const half_t* beta, float eps, int rd_mean, hipStream_t st) {
    if (r <= 1) launch_tile<LPR, 1, MODE>(batch, n, m, mat, out, alpha, beta, eps, rd_mean, st);
    else if (r <= 2) launch_tile<LPR, 2, MODE>(batch, n, m, mat, out, alpha, beta, eps, rd_mean, st);
    else if (r <= 4) launch_tile<LPR, 4, MODE>(batch, n, m, mat, out, alpha, beta, eps, rd_mean, st);
    else if (r <= 8) launch_tile<LPR, 8, MODE>(batch, n, m, mat, out, alpha, beta, eps, rd_mean, st);
    else return false;
    return true;
}

// `fixed` == nullptr: team launches take their packet slots from the library's pool (exchange.hip).
// Otherwise the one team launch a call may need uses the slots, counters and status word `fixed`
// names (fixed_slots of them) and a shape that needs more is refused with CPMK_ETOOBIG.
static int layernorm_dispatch(int32_t batch, int32_t n, int32_t m, const void* mat, void* out, const void* alpha,
                              const void* beta, float eps, int rd_mean, hipStream_t st, const XchLaunch* fixed = nullptr,
                              int64_t fixed_slots = 0) {
    if (batch < 0 || n < 0 || m < 0) return CPMK_EBADARG;
    if ((int64_t)batch * n * m == 0) return 0;
    if (any_null(mat, out)) return CPMK_EBADARG;
    const half_t* x = (const half_t*)mat;
    half_t* y = (half_t*)out;
    const half_t* al = (const half_t*)alpha;
    const half_t* be = (const half_t*)beta;
    if (m == 1 && alpha == nullptr) {
        hipLaunchKernelGGL(k_layernorm_rows, dim3((unsigned)batch), dim3(256), 0, st, n, x, y, eps, rd_mean);
        return launch_status();
    }
    // rows of whole 16-byte pieces in 16-byte aligned buffers: 16-byte accesses; any other width or alignment: the same
    // kernels (64-column tiles only) moving their tiles element by element
    const bool wide = m % 8 == 0 && aligned16(mat) && aligned16(out);
    // the 128-byte row segments of the 64-column tiles are whole cache lines: the non-temporal hint pays there only
    const bool lines = m % 64 == 0 && (reinterpret_cast<uintptr_t>(mat) & 127u) == 0 && (reinterpret_cast<uintptr_t>(out) & 127u) == 0;
    if ((int64_t)n * m < (1ll << 31) && (wide || m > 1)) {
        // widest row segment whose tile still fits the register budget (at most 8 pieces per lane)
        bool ok = false;
        if (n > 128 * 8 && (m >= 64 || !wide)) {
            // tall columns: 64-column tiles, the rows split over a team of workgroups
            const int64_t tiles = ceil_div(m, 64);
            // 1024 rows a part (one 1024-thread workgroup per compute unit) while those parts fit the chip in
            // one round; with more rounds, or shorter columns, 512 rows a part: two workgroups share a compute
            // unit and one's loads overlap the other's exchange and stores (16 x 4096 x 1024: 66 -> 60 us;
            // the one-round 8 x 4096 x 512 is 0.6 us faster with the large parts)
            const bool big = n >= 2048 && (n > 4096 || tiles * batch * ceil_div(n, 1024) <= compute_units());
            const int64_t parts = ceil_div(n, big ? 1024 : 512);
            if (fixed != nullptr && parts <= kXchMaxParts && tiles * parts * batch > fixed_slots) return CPMK_ETOOBIG;
            if (parts <= kXchMaxParts && tiles * parts <= kXchSlots) {
                // one packet slot per (team, part): batches beyond the pool go out in several launches
                const int64_t per_launch = fixed != nullptr ? batch : kXchSlots / (tiles * parts);
                bool no_slots = false;
                for (int64_t b0 = 0; b0 < batch && !no_slots; b0 += per_launch) {
                    const int64_t nb = batch - b0 < per_launch ? batch - b0 : per_launch;
                    XchScope xs;
                    if (fixed != nullptr) {
                        xs.xl = *fixed;
                    } else {
                        const int rc = xs.begin(tiles * nb * parts, st);
                        if (rc == kXchFull && b0 == 0) {
                            no_slots = true;       // recorded into a graph and the capture reserve is used up: the kernel without packets below
                            break;
                        }
                        if (rc != 0) return rc == kXchFull ? CPMK_ETOOBIG : rc;
                    }
                    const XchLaunch& xl = xs.xl;
                    const dim3 grid((unsigned)xch_team_grid(tiles * nb, parts));
                    const half_t* xb = x + b0 * n * m;
                    half_t* yb = y + b0 * n * m;
                    auto go = [&](auto kern, int threads) {
                        hipLaunchKernelGGL(kern, grid, dim3(threads), 0, st, n, m, (int32_t)tiles, (int32_t)parts, xb, yb, al, be, eps,
                                           rd_mean, (uint32_t)(tiles * nb), xl);
                    };
                    auto pick = [&](auto modec) {
                        constexpr int MODE = decltype(modec)::value;
                        if (big) {
                            if (al != nullptr) go(k_layernorm_team<1024, 8, true, MODE>, 1024);
                            else go(k_layernorm_team<1024, 8, false, MODE>, 1024);
                        } else {
                            if (al != nullptr) go(k_layernorm_team<512, 8, true, MODE>, 512);
                            else go(k_layernorm_team<512, 8, false, MODE>, 512);
                        }
                    };
                    if (!wide) pick(std::integral_constant<int, 2>{});
                    else if (lines) pick(std::integral_constant<int, 0>{});
                    else pick(std::integral_constant<int, 1>{});
                    const int e = launch_status();
                    const int rc2 = xs.end();
                    if (e != 0 || rc2 != 0) return e ? e : rc2;
                }
                if (!no_slots) return 0;
            }
        }
        if (!wide) ok = n <= 128 * 8 && launch_tile_r<8, 2>((int)ceil_div(n, 128), batch, n, m, x, y, al, be, eps, rd_mean, st);
        else if (n <= 128 * 8 && m >= 64 && !lines) ok = launch_tile_r<8, 1>((int)ceil_div(n, 128), batch, n, m, x, y, al, be, eps, rd_mean, st);
        else if (n <= 128 * 8 && m >= 64) ok = launch_tile_r<8>((int)ceil_div(n, 128), batch, n, m, x, y, al, be, eps, rd_mean, st);
        else if (n <= 256 * 8 && m >= 32) ok = launch_tile_r<4>((int)ceil_div(n, 256), batch, n, m, x, y, al, be, eps, rd_mean, st);
        else ok = launch_tile_r<2>((int)ceil_div(n, 512), batch, n, m, x, y, al, be, eps, rd_mean, st);
        if (ok) return launch_status();
    }
    // the batch is the grid's y dimension (at most 65535): larger batches go out in several launches
    for (int64_t b0 = 0; b0 < batch; b0 += 65535) {
        const int64_t nb = batch - b0 < 65535 ? batch - b0 : 65535;
        hipLaunchKernelGGL(k_layernorm_generic, dim3((unsigned)ceil_div(m, 64), (unsigned)nb), dim3(256), 0, st, n, m,
                           x + b0 * n * m, y + b0 * n * m, al, be, eps, rd_mean);
        if (int e = launch_status()) return e;
    }
    return 0;
}

// ---------------------------------------------------------------------------------------
// Packet slots of cpmk_layernorm_forward_noalloc: kNoAllocSlots slots of kXchVals packets, then
// one retire counter per slot.  Static storage, so every GPU the library runs on holds its own
// copy (2.1 MB) at its own address until the process ends.  All zero at load; a team launch
// leaves it all zero again (the last member of each team clears the team's slots and counter).
constexpr int kNoAllocSlots = 2048;
static __device__ __align__(256) uint64_t scratch[(size_t)kNoAllocSlots * kXchVals + kNoAllocSlots];

// The array's address on the current device, looked up once per device (`scratch` itself is only a
// host-side handle for the symbol, not a device address).
static int noalloc_scratch(uint64_t** out) {
    static std::mutex mu;
    static uint64_t* ptr[64] = {nullptr};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= 64) return CPMK_EBADARG;
    std::lock_guard<std::mutex> lock(mu);
    if (ptr[dev] == nullptr) {
        uint64_t* p = nullptr;
        e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (p == nullptr) return CPMK_EBADARG;
        ptr[dev] = p;
    }
    *out = ptr[dev];
    return 0;
}

}  // namespace cpmk

using namespace cpmk;

extern "C" {

int cpmk_layernorm_forward(int32_t batch, int32_t n, int32_t m, const void* mat, void* out, float eps,
                           int rd_mean, void* stream) {
    clear_stale_error();
    return layernorm_dispatch(batch, n, m, mat, out, nullptr, nullptr, eps, rd_mean, (hipStream_t)stream);
}

int cpmk_layernorm_forward_noalloc(int32_t batch, int32_t n, int32_t m, const void* mat, void* out, float eps,
                                   int rd_mean, void* stream) {
    clear_stale_error();
    uint64_t* base = nullptr;
    if (int rc = noalloc_scratch(&base)) return rc;
    XchLaunch xl;
    xl.region = base;
    xl.counters = base + (size_t)kNoAllocSlots * kXchVals;
    xl.tag = xch_next_tag();
    xl.first = -1;
    if (int rc = xch_status_words(&xl.status, &xl.host_status)) return rc;
    return layernorm_dispatch(batch, n, m, mat, out, nullptr, nullptr, eps, rd_mean, (hipStream_t)stream, &xl, kNoAllocSlots);
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
    if (any_null(mat, out)) return CPMK_EBADARG;
    hipLaunchKernelGGL(k_layernorm_rows, dim3((unsigned)batch), dim3(256), 0, (hipStream_t)stream, n,
                       (const half_t*)mat, (half_t*)out, eps, rd_mean);
    return launch_status();
}

}  // extern "C"
