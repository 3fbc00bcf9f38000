// Softmax over dim 1 of (batch, n, m) fp16 and over contiguous rows (decode step):
//   M = max(max_i x, -1e6);  S = sum_i exp(x - M) + 1e-10;  out = fp16(exp(x - M) / S)
// (cuda/softmax.cu:6-43, :117-159).  A column that is entirely -inf therefore yields 0, not
// NaN.  The reference reads the input three times and evaluates expf twice per element; the
// tile kernels below read once, evaluate exp once and keep the results in registers:
//   k_softmax_tile    one column tile per workgroup
//   k_softmax_stream  many tiles per compute unit: persistent workgroups, next tile prefetched into
//                     LDS by DMA, tiles handed out from a device-side counter
//   k_softmax_team    columns too tall for one workgroup, shared by a team
//   k_softmax_generic any shape;  k_softmax_rows  contiguous rows (decode step)
#include "dim1.h"
#include "exchange.h"

namespace cpmk {

constexpr float kLog2e = 1.4426950408889634f;

// exp(x - M) as one fma and one v_exp_f32: exp2(x*log2e - M*log2e).
__device__ inline float exp_shift(float x, float mlog2e) { return __builtin_amdgcn_exp2f(__builtin_fmaf(x, kLog2e, -mlog2e)); }

// The softmax of the columns of one register-resident tile, in place in v (rows past n hold -inf).
template <int NT, int LPR, int R>
__device__ __forceinline__ void softmax_cols(half8_t (&v)[R], float* lds) {
    half8_t hm = v[0];
#pragma unroll
    for (int p = 1; p < R; ++p) hm = __builtin_elementwise_max(hm, v[p]);
    float mx[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) mx[e] = (float)hm[e];
    coltile_reduce<NT, LPR, 1, true>(mx, lds);

    float ex[R][8], s[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        mx[e] = fmaxf(mx[e], -1e6f) * kLog2e;
        s[e] = 0.0f;
    }
#pragma unroll
    for (int p = 0; p < R; ++p) {
        const uint4_t raw = __builtin_bit_cast(uint4_t, v[p]);
        const bool all_ninf = (raw.x == 0xfc00fc00u) & (raw.y == 0xfc00fc00u) & (raw.z == 0xfc00fc00u) & (raw.w == 0xfc00fc00u);
        if (__builtin_amdgcn_ballot_w64(!all_ninf) == 0) {      // wave-uniform: nothing but -inf here
#pragma unroll
            for (int e = 0; e < 8; ++e) ex[p][e] = 0.0f;
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                ex[p][e] = exp_shift((float)v[p][e], mx[e]);   // rows >= n hold -inf -> 0
                s[e] += ex[p][e];
            }
        }
    }
    coltile_reduce<NT, LPR, 1, false>(s, lds);
#pragma unroll
    for (int e = 0; e < 8; ++e) s[e] = 1.0f / (s[e] + 1e-10f);
#pragma unroll
    for (int p = 0; p < R; ++p)
#pragma unroll
        for (int e = 0; e < 8; ++e) v[p][e] = round_f16(ex[p][e] * s[e]);
}

// Register-resident column tile: HBM is read once and exp is evaluated once per element.  The
// kernel is co-limited by HBM and by the VALU (v_exp_f32 is a quarter-rate instruction), so the
// arithmetic is kept lean: column maxima on the packed fp16 inputs (exact), one fused
// multiply-add and one exp2 per element, and a 16-byte piece whose 8 inputs are all -inf for
// every lane of the wave (whole rows masked out, as in causal attention) is skipped -- its
// exponentials are exactly 0.
// MODE 0: 16-byte accesses, non-temporal where a tile's row segments are whole cache lines; 1: 16-byte accesses without
// the hint (rows that do not start on 128-byte boundaries); 2: any m and alignment, element by element (dim1.h).
template <int NT, int LPR, int R, int MODE = 0>
__global__ __launch_bounds__(NT) void k_softmax_tile(int32_t n, int32_t m, int32_t tiles_per_batch,
                                                     const half_t* inp, half_t* out) {
    using T = ColTile<NT, LPR, R>;
    __shared__ float lds[(T::NW + 1) * T::COLS];
    const uint32_t t = xcd_remap(blockIdx.x, gridDim.x);
    const uint32_t b = t / tiles_per_batch, ct = t - b * tiles_per_batch;
    const int32_t col0 = ct * T::COLS + (threadIdx.x % LPR) * 8;
    const int64_t boff = (int64_t)b * n * m;

    half8_t v[R];
    coltile_load<NT, LPR, R, LPR == 8 && MODE == 0, MODE == 2>(v, inp + boff, n, m, col0, (half_t)(-__builtin_inff()));

    softmax_cols<NT, LPR, R>(v, lds);
    coltile_store<NT, LPR, R, LPR == 8 && MODE == 0, MODE == 2>(v, out + boff, n, m, col0);
}

// The same for many tiles per compute unit: persistent workgroups, each wave fetching its share
// of the NEXT tile straight into LDS (global_load_lds, 1 KB per wave instruction, no registers)
// while the current tile is reduced, exponentiated and stored.  A lane reads back exactly the 16
// bytes it requested, so the staging needs no barrier, only the wave's own vmcnt; the wait sits
// in front of the current tile's stores, where the loads issued a whole compute phase earlier
// have landed, and the stores then drain under the next tile.  Loads and stores carry the
// non-temporal hint (512 x 1024 x 1024: 396 -> 385 us; a plain copy of that size gains 10 % from it).
//
// Tiles are handed out dynamically: the first gridDim.x tiles by workgroup index, the rest from a
// counter in device memory.  With a fixed share per workgroup the kernel ends with its slowest
// compute unit, and on this chip one in eight gets 25 % less memory bandwidth than the rest.
// The two counters (sched[0]: tiles handed out beyond the first round, sched[1]: finished workgroups) are the
// launch's own: they come out of the exchange pool (exchange.h) with the same bookkeeping as a team's packet
// slots, so no other launch or graph that may run at the same time shares them.  The workgroup that finishes
// last clears them, so the next holder (or a replay of the graph) finds them zero.

template <int NT, int LPR, int R>
__global__ __launch_bounds__(NT) void k_softmax_stream(int32_t n, int32_t m, int32_t tiles_per_batch, uint32_t ntiles, unsigned int* sched,
                                                       const half_t* inp, half_t* out) {
    using T = ColTile<NT, LPR, R>;
    constexpr int RPP = NT / LPR;
    extern __shared__ __attribute__((aligned(16))) int8_t dyn[];        // NT*R*16 bytes of staging, the reduction scratch, one word for the next tile
    float* lds = reinterpret_cast<float*>(dyn + NT * R * 16);
    uint32_t* s_next = reinterpret_cast<uint32_t*>(lds + (T::NW + 1) * T::COLS);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int8_t* stage = dyn + wave * (R * 1024) + lane * 16;
    const uint32_t stage_addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) int8_t*)(dyn + wave * (R * 1024));
    const uint32_t G = gridDim.x;
    unsigned int* ctr = sched;
    const int rg = tid / LPR, cg = tid % LPR;
    auto issue = [&](uint32_t t) __attribute__((always_inline)) {
        const uint32_t b = t / tiles_per_batch, ct = t - b * tiles_per_batch;
        const int32_t cc = min((int32_t)(ct * T::COLS + cg * 8), m - 8);          // clamped: lanes past the edge are refilled below
        const int8_t* base = reinterpret_cast<const int8_t*>(inp + (int64_t)b * n * m);
#pragma unroll
        for (int p = 0; p < R; ++p) {
            const int32_t row = min(p * RPP + rg, n - 1);
            lds_dma16_nt(((uint32_t)row * (uint32_t)m + (uint32_t)cc) * 2u, base, stage_addr + p * 1024);
        }
    };
    uint32_t t = blockIdx.x;                       // gridDim.x <= ntiles
    issue(t);
    if (tid == 0) *s_next = G + atomicAdd(ctr, 1u);
    wait_vmcnt<0>();
    __syncthreads();
    uint32_t tn = __builtin_amdgcn_readfirstlane(*s_next);
    while (t < ntiles) {
        const uint32_t b = t / tiles_per_batch, ct = t - b * tiles_per_batch;
        const int32_t col0 = ct * T::COLS + cg * 8;
        const int64_t boff = (int64_t)b * n * m;
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        half8_t v[R];
#pragma unroll
        for (int p = 0; p < R; ++p) {
            half8_t x = *reinterpret_cast<const half8_t*>(stage + p * 1024);
            if (!(p * RPP + rg < n && col0 < m)) {
#pragma unroll
                for (int e = 0; e < 8; ++e) x[e] = (half_t)(-__builtin_inff());
            }
            v[p] = x;
        }
#pragma unroll
        for (int p = 0; p < R; ++p) asm volatile("" : "+v"(v[p]));      // the reads are done before the staging is refilled
        __builtin_amdgcn_sched_barrier(0);
        if (tn < ntiles) issue(tn);
        uint32_t after = 0;
        if (tid == 0) after = G + atomicAdd(ctr, 1u);                   // the tile after the next; used only after the arithmetic
        __builtin_amdgcn_sched_barrier(0);
        softmax_cols<NT, LPR, R>(v, lds);
        __builtin_amdgcn_sched_barrier(0);
        wait_vmcnt<0>();            // the next tile has landed; the previous tile's stores finished long ago
        if (tid == 0) *s_next = after;
        __syncthreads();
        const uint32_t tnn = __builtin_amdgcn_readfirstlane(*s_next);
        __builtin_amdgcn_sched_barrier(0);
        coltile_store<NT, LPR, R, true>(v, out + boff, n, m, col0);
        t = tn;
        tn = tnn;
    }
    // every workgroup is past its last fetch when it signs off, so the last one to do so may clear the counters
    if (tid == 0) {
        if (atomicAdd(sched + 1, 1u) == G - 1) {
            atomicExch(sched, 0u);
            atomicExch(sched + 1, 0u);
        }
    }
}

// Columns too tall for one workgroup's registers at 128-byte row segments: the n rows of a
// 64-column tile are split over a team of `parts` workgroups (exchange.h).  Each computes, for its own rows, the column maximum m_p (floored at
// -1e6 like M itself) and the exponentials and their sum s_p relative to m_p, posts (m_p, s_p),
// and rescales by exp(m_p - M) / S with M = max_p m_p and S = sum_p s_p exp(m_p - M) + 1e-10,
// which is the single-workgroup result up to two extra fp32 roundings.
template <int NT, int R, int MODE = 0>
__global__ __launch_bounds__(NT) void k_softmax_team(int32_t n, int32_t m, int32_t tiles_per_batch, int32_t parts,
                                                     const half_t* inp, half_t* out, uint32_t nteams, XchLaunch xl) {
    constexpr int LPR = 8;
    using T = ColTile<NT, LPR, R>;
    static_assert(T::COLS * 2 == kXchVals, "slot layout");
    uint64_t* const xch = xl.region;
    const uint32_t tag = xl.tag;
    __shared__ float lds[(T::NW + 1) * T::COLS];
    __shared__ float tot[kXchVals];
    const int tid = threadIdx.x;
    XchMember me;
    if (!xch_member(blockIdx.x, parts, nteams, me)) return;
    const uint32_t part = me.part, team = me.team;
    const uint32_t b = team / tiles_per_batch, ct = team - b * tiles_per_batch;
    const int32_t col0 = ct * T::COLS + (tid % LPR) * 8;
    const int32_t own0 = part * T::ROWS;
    const int32_t own_n = min(T::ROWS, n - own0);
    const int64_t boff = (int64_t)b * n * m + (int64_t)own0 * m;

    half8_t v[R];
    coltile_load<NT, LPR, R, MODE == 0, MODE == 2>(v, inp + boff, own_n, m, col0, (half_t)(-__builtin_inff()));

    half8_t hm = v[0];
#pragma unroll
    for (int p = 1; p < R; ++p) hm = __builtin_elementwise_max(hm, v[p]);
    float mx[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) mx[e] = (float)hm[e];
    coltile_reduce<NT, LPR, 1, true>(mx, lds);

    float ex[R][8], s[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        mx[e] = fmaxf(mx[e], -1e6f) * kLog2e;       // m_p, in units of log2(e)
        s[e] = 0.0f;
    }
#pragma unroll
    for (int p = 0; p < R; ++p) {
        const uint4_t raw = __builtin_bit_cast(uint4_t, v[p]);
        const bool all_ninf = (raw.x == 0xfc00fc00u) & (raw.y == 0xfc00fc00u) & (raw.z == 0xfc00fc00u) & (raw.w == 0xfc00fc00u);
        if (__builtin_amdgcn_ballot_w64(!all_ninf) == 0) {
#pragma unroll
            for (int e = 0; e < 8; ++e) ex[p][e] = 0.0f;
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                ex[p][e] = exp_shift((float)v[p][e], mx[e]);
                s[e] += ex[p][e];
            }
        }
    }
    coltile_reduce<NT, LPR, 1, false>(s, lds);

    // packet c: m_p of tile column c; packet 64 + c: s_p
    uint64_t* team_slots = xch + (size_t)team * parts * kXchVals;
    if (tid < LPR) {
        uint64_t* slot = team_slots + (size_t)part * kXchVals;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            xch_post(slot, tid * 8 + e, mx[e], tag);
            xch_post(slot, T::COLS + tid * 8 + e, s[e], tag);
        }
    }
    if (tid < T::COLS) {
        const uint64_t deadline = wall_clock64() + kXchTimeoutTicks;
        static_assert(kXchMaxParts == 8, "two rounds of gathers cover a team");
        float mp[kXchMaxParts], sp[kXchMaxParts];
        bool ok = true;
#pragma unroll
        for (int q0 = 0; q0 < kXchMaxParts; q0 += 4) {          // four parts' m_p, then their s_p, per round trip (all eight at once, or both statistics at once, spill registers)
            float a[4], c[4];
            ok &= xch_gather<4>(team_slots, parts, q0, tid, tag, deadline, a);
            ok &= xch_gather<4>(team_slots, parts, q0, T::COLS + tid, tag, deadline, c);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                mp[q0 + j] = q0 + j < parts ? a[j] : -__builtin_inff();        // (absent parts: s_p is 0 already)
                sp[q0 + j] = c[j];
            }
        }
        float M = -__builtin_inff();
#pragma unroll
        for (int q = 0; q < kXchMaxParts; ++q) M = fmaxf(M, mp[q]);
        float S = 0.0f;
#pragma unroll
        for (int q = 0; q < kXchMaxParts; ++q)
            if (q < parts) S += sp[q] * __builtin_amdgcn_exp2f(mp[q] - M);
        tot[tid] = M;
        tot[T::COLS + tid] = ok ? 1.0f / (S + 1e-10f) : __builtin_nanf("");
        if (!ok) xch_flag(xl, kXchStatusTimeout);
    }
    __syncthreads();
    const int cg = tid % LPR;
    float f[8];
#pragma unroll
    for (int e = 0; e < 8; ++e)
        f[e] = __builtin_amdgcn_exp2f(mx[e] - tot[cg * 8 + e]) * tot[T::COLS + cg * 8 + e];     // exp(m_p - M) / S
#pragma unroll
    for (int p = 0; p < R; ++p)
#pragma unroll
        for (int e = 0; e < 8; ++e) v[p][e] = round_f16(ex[p][e] * f[e]);
    coltile_store<NT, LPR, R, MODE == 0, MODE == 2>(v, out + boff, own_n, m, col0);
    if (tid < 64) xch_retire(xl, team, parts);     // after the barrier above: this workgroup holds all it needs
}

// Generic fallback: 64 columns x 4 row groups, three passes (max, sum, write).  All reads of
// a column by other threads finish before the barrier that precedes the first store, and
// the last pass re-reads each element in the thread that overwrites it: out may alias inp.
__global__ __launch_bounds__(256) void k_softmax_generic(int32_t n, int32_t m, const half_t* inp, half_t* out) {
    __shared__ float red[4][64];
    const int c = threadIdx.x & 63, rg = threadIdx.x >> 6;
    const int32_t col = blockIdx.x * 64 + c;
    const int64_t boff = (int64_t)blockIdx.y * n * m;
    float mx = -__builtin_inff();
    if (col < m)
        for (int32_t i = rg; i < n; i += 4) mx = fmaxf(mx, (float)inp[boff + (int64_t)i * m + col]);
    red[rg][c] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red[0][c], red[1][c]), fmaxf(red[2][c], red[3][c]));
    mx = fmaxf(mx, -1e6f) * kLog2e;
    __syncthreads();
    float s = 0.0f;
    if (col < m)
        for (int32_t i = rg; i < n; i += 4) s += exp_shift((float)inp[boff + (int64_t)i * m + col], mx);
    red[rg][c] = s;
    __syncthreads();
    s = 1.0f / (red[0][c] + red[1][c] + red[2][c] + red[3][c] + 1e-10f);
    if (col < m)
        for (int32_t i = rg; i < n; i += 4) {
            const int64_t o = boff + (int64_t)i * m + col;
            out[o] = round_f16(exp_shift((float)inp[o], mx) * s);
        }
}

// Contiguous rows (batch, n), in place capable: one 256-thread workgroup per row.
__global__ __launch_bounds__(256) void k_softmax_rows(int32_t n, const half_t* inp, half_t* out) {
    __shared__ float red[4];
    const half_t* p = inp + (int64_t)blockIdx.x * n;
    half_t* o = out + (int64_t)blockIdx.x * n;
    float mx = -__builtin_inff();
    for (int32_t i = threadIdx.x; i < n; i += 256) mx = fmaxf(mx, (float)p[i]);
    mx = fmaxf(block_max<4>(mx, red), -1e6f) * kLog2e;
    float s = 0.0f;
    for (int32_t i = threadIdx.x; i < n; i += 256) s += exp_shift((float)p[i], mx);
    s = 1.0f / (block_sum<4>(s, red) + 1e-10f);
    for (int32_t i = threadIdx.x; i < n; i += 256) o[i] = round_f16(exp_shift((float)p[i], mx) * s);
}

template <int NT, int LPR, int R, int MODE>
static void launch_tile(int32_t batch, int32_t n, int32_t m, const half_t* inp, half_t* out, hipStream_t st) {
    const int32_t tiles = (int32_t)ceil_div(m, LPR * 8);
    hipLaunchKernelGGL((k_softmax_tile<NT, LPR, R, MODE>), dim3((unsigned)((int64_t)tiles * batch)), dim3(NT), 0, st, n, m,
                       tiles, inp, out);
}

// persistent variant: one workgroup per compute unit, 16 bytes of LDS staging per element slot.  Returns kXchFull
// (and launches nothing) when the call is recorded into a graph and the pool's capture reserve has no room
// for the launch's counters: the caller then records a kernel that needs none.
template <int NT, int LPR, int R>
static int launch_stream(int32_t batch, int32_t n, int32_t m, const half_t* inp, half_t* out, hipStream_t st) {
    using T = ColTile<NT, LPR, R>;
    constexpr int smem = NT * R * 16 + (T::NW + 1) * T::COLS * (int)sizeof(float) + 16;
    static_assert(smem <= 160 * 1024, "LDS of one compute unit");
    auto kern = k_softmax_stream<NT, LPR, R>;
    static std::atomic<bool> lds_enabled[64];
    if (int e = enable_dynamic_lds(reinterpret_cast<const void*>(kern), smem, lds_enabled)) return e;
    const int32_t tiles = (int32_t)ceil_div(m, LPR * 8);
    const int64_t ntiles = (int64_t)tiles * batch;
    const int cus = compute_units();
    XchScope xs;
    if (int rc = xs.begin(1, st)) return rc;
    // the first team counter of the launch's range: eight bytes, all zero, used as two 32-bit counters
    hipLaunchKernelGGL(kern, dim3((unsigned)(ntiles < cus ? ntiles : cus)), dim3(NT), smem, st, n, m, tiles, (uint32_t)ntiles,
                       reinterpret_cast<unsigned int*>(xs.xl.counters), inp, out);
    const int e = launch_status();
    const int rc2 = xs.end();
    return e ? e : rc2;
}

template <int NT, int LPR, int MODE>
static bool launch_tile_r(int r, int32_t batch, int32_t n, int32_t m, const half_t* inp, half_t* out,
                          hipStream_t st) {
    if (r <= 1) launch_tile<NT, LPR, 1, MODE>(batch, n, m, inp, out, st);
    else if (r <= 2) launch_tile<NT, LPR, 2, MODE>(batch, n, m, inp, out, st);
    else if (r <= 4) launch_tile<NT, LPR, 4, MODE>(batch, n, m, inp, out, st);
    else if (r <= 8) launch_tile<NT, LPR, 8, MODE>(batch, n, m, inp, out, st);
    else return false;
    return true;
}

// columns taller than this go to the team kernel (single workgroups hold up to 2048 rows at 64-byte row segments)
constexpr int32_t kSoftmaxTeamMin = 2048;

static int softmax_dispatch(int32_t batch, int32_t n, int32_t m, const void* inp, void* out, hipStream_t st) {
    if (batch < 0 || n < 0 || m < 0) return CPMK_EBADARG;
    if ((int64_t)batch * n * m == 0) return 0;
    if (any_null(inp, out)) return CPMK_EBADARG;
    const half_t* x = (const half_t*)inp;
    half_t* y = (half_t*)out;
    if (m == 1) {
        hipLaunchKernelGGL(k_softmax_rows, dim3((unsigned)batch), dim3(256), 0, st, n, x, y);
        return launch_status();
    }
    // rows of whole 16-byte pieces in 16-byte aligned buffers: 16-byte accesses, with the non-temporal hint where the
    // 128-byte row segments of the 64-column tiles are whole cache lines; any other width or alignment: the same kernels
    // moving their tiles element by element
    const bool wide = m % 8 == 0 && aligned16(inp) && aligned16(out);
    const bool lines = wide && m % 64 == 0 && (reinterpret_cast<uintptr_t>(inp) & 127u) == 0 && (reinterpret_cast<uintptr_t>(out) & 127u) == 0;
    auto with_mode = [&](auto&& f) {       // f(integral_constant<int, MODE>)
        if (!wide) return f(std::integral_constant<int, 2>{});
        if (lines) return f(std::integral_constant<int, 0>{});
        return f(std::integral_constant<int, 1>{});
    };
    if ((int64_t)n * m < (1ll << 31)) {
        bool ok = false;
        if (n > kSoftmaxTeamMin && m >= 64) {
            const int64_t tiles = ceil_div(m, 64);
            const int64_t parts = ceil_div(n, 1024);          // 1024 rows a part
            if (parts <= kXchMaxParts && tiles * parts <= kXchSlots) {
                // one packet slot per (team, part): batches beyond the pool go out in several launches
                const int64_t per_launch = kXchSlots / (tiles * parts);
                bool no_slots = false;
                for (int64_t b0 = 0; b0 < batch; b0 += per_launch) {
                    const int64_t nb = batch - b0 < per_launch ? batch - b0 : per_launch;
                    XchScope xs;
                    const int rc = xs.begin(tiles * nb * parts, st);
                    if (rc == kXchFull && b0 == 0) {
                        no_slots = true;       // recorded into a graph and the capture reserve is used up: a kernel without packets below
                        break;
                    }
                    if (rc != 0) return rc == kXchFull ? CPMK_ETOOBIG : rc;
                    const dim3 grid((unsigned)xch_team_grid(tiles * nb, parts));
                    const half_t* xb = x + b0 * n * m;
                    half_t* yb = y + b0 * n * m;
                    with_mode([&](auto mc) {
                        hipLaunchKernelGGL((k_softmax_team<1024, 8, decltype(mc)::value>), grid, dim3(1024), 0, st, n, m, (int32_t)tiles,
                                           (int32_t)parts, xb, yb, (uint32_t)(tiles * nb), xs.xl);
                        return true;
                    });
                    const int e = launch_status();
                    const int rc2 = xs.end();
                    if (e != 0 || rc2 != 0) return e ? e : rc2;
                }
                if (!no_slots) return 0;
            }
        }
        // several tiles per compute unit: the persistent kernel keeps loads in flight during the arithmetic
        if (lines && n > 256 && n <= 1024 && m >= 64 && ceil_div(m, 64) * batch >= 2 * (int64_t)compute_units() &&
            ceil_div(m, 64) * batch < (1ll << 31)) {
            const int rc = n > 512 ? launch_stream<1024, 8, 8>(batch, n, m, x, y, st) : launch_stream<1024, 8, 4>(batch, n, m, x, y, st);
            if (rc != kXchFull) return rc;
        }
        ok = with_mode([&](auto mc) {
            constexpr int MODE = decltype(mc)::value;
            if (n <= 64 * 8 && m >= 64) return launch_tile_r<512, 8, MODE>((int)ceil_div(n, 64), batch, n, m, x, y, st);
            if (n <= 128 * 8 && m >= 64) return launch_tile_r<1024, 8, MODE>((int)ceil_div(n, 128), batch, n, m, x, y, st);
            if (n <= 256 * 8 && m >= 32) return launch_tile_r<1024, 4, MODE>((int)ceil_div(n, 256), batch, n, m, x, y, st);
            if (n <= 512 * 8) return launch_tile_r<1024, 2, MODE>((int)ceil_div(n, 512), batch, n, m, x, y, st);
            return false;
        });
        if (ok) return launch_status();
    }
    // the batch is the grid's y dimension (at most 65535): larger batches go out in several launches
    for (int64_t b0 = 0; b0 < batch; b0 += 65535) {
        const int64_t nb = batch - b0 < 65535 ? batch - b0 : 65535;
        hipLaunchKernelGGL(k_softmax_generic, dim3((unsigned)ceil_div(m, 64), (unsigned)nb), dim3(256), 0, st, n, m,
                           x + b0 * n * m, y + b0 * n * m);
        if (int e = launch_status()) return e;
    }
    return 0;
}

}  // namespace cpmk

using namespace cpmk;

extern "C" {

int cpmk_softmax_forward(int32_t batch, int32_t n, int32_t m, const void* inp, void* out, void* stream) {
    clear_stale_error();
    return softmax_dispatch(batch, n, m, inp, out, (hipStream_t)stream);
}

int cpmk_softmax_step_inplace(int32_t batch, int32_t n, void* x, void* stream) {
    clear_stale_error();
    if (batch < 0 || n < 0) return CPMK_EBADARG;
    if ((int64_t)batch * n == 0) return 0;
    if (x == nullptr) return CPMK_EBADARG;
    hipLaunchKernelGGL(k_softmax_rows, dim3((unsigned)batch), dim3(256), 0, (hipStream_t)stream, n,
                       (const half_t*)x, (half_t*)x);
    return launch_status();
}

}  // extern "C"
