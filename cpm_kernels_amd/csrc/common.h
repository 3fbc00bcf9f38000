// Shared device/host helpers for the gfx950 kernels of libcpmk_hip.so.
// Everything here assumes 64-wide wavefronts (CDNA); nothing is written for 32-lane warps.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <atomic>
#include "../../include/cpmk.h"

namespace cpmk {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));

typedef float float4_t __attribute__((ext_vector_type(4)));
typedef int32_t int4_t __attribute__((ext_vector_type(4)));
typedef int32_t int2_t __attribute__((ext_vector_type(2)));
typedef int32_t int16_tv __attribute__((ext_vector_type(16)));
typedef float float16_tv __attribute__((ext_vector_type(16)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));

// Wide accesses at addresses that are not multiples of their size: global loads and stores of this target need no
// alignment (the compiler itself emits 16-byte accesses for data declared with alignment 1); an access that crosses
// a cache line costs a second request.  Eight halves at any half's address, eight bytes at any address:
struct __attribute__((packed, aligned(2))) Half8Any { uint32_t x, y, z, w; };
struct __attribute__((packed, aligned(1))) Byte8Any { uint32_t x, y; };
__device__ __forceinline__ half8_t load_half8_any(const half_t* p) { return __builtin_bit_cast(half8_t, *reinterpret_cast<const Half8Any*>(p)); }
__device__ __forceinline__ void store_half8_any(half_t* p, half8_t v) { *reinterpret_cast<Half8Any*>(p) = __builtin_bit_cast(Half8Any, v); }
__device__ __forceinline__ void store_byte8_any(int8_t* p, uint32_t lo, uint32_t hi) { *reinterpret_cast<Byte8Any*>(p) = Byte8Any{lo, hi}; }

// The first t (1..7, the same for the whole wave) of eight halves at p, at any address, in at most three accesses
// (8, 4 and 2 bytes); the other elements of the result keep `r`'s values.
struct __attribute__((packed, aligned(2))) Half4Any { uint32_t x, y; };
struct __attribute__((packed, aligned(2))) Half2Any { uint32_t x; };
__device__ __forceinline__ half8_t load_half8_head_any(const half_t* p, int t, half8_t r) {
    if (t & 4) {
        const half4_t q = __builtin_bit_cast(half4_t, *reinterpret_cast<const Half4Any*>(p));
        r[0] = q[0]; r[1] = q[1]; r[2] = q[2]; r[3] = q[3];
    }
    if (t & 2) {
        const half2_t q = __builtin_bit_cast(half2_t, *reinterpret_cast<const Half2Any*>(p + (t & 4)));
        if (t & 4) { r[4] = q[0]; r[5] = q[1]; } else { r[0] = q[0]; r[1] = q[1]; }
    }
    if (t & 1) {
        const half_t h = p[t & 6];
        if ((t & 6) == 0) r[0] = h;
        else if ((t & 6) == 2) r[2] = h;
        else if ((t & 6) == 4) r[4] = h;
        else r[6] = h;
    }
    return r;
}
__device__ __forceinline__ void store_half8_head_any(half_t* p, int t, half8_t v) {
    if (t & 4) *reinterpret_cast<Half4Any*>(p) = __builtin_bit_cast(Half4Any, half4_t{v[0], v[1], v[2], v[3]});
    if (t & 2) {
        const half2_t q = (t & 4) ? half2_t{v[4], v[5]} : half2_t{v[0], v[1]};
        *reinterpret_cast<Half2Any*>(p + (t & 4)) = __builtin_bit_cast(Half2Any, q);
    }
    if (t & 1) p[t & 6] = (t & 6) == 0 ? v[0] : (t & 6) == 2 ? v[2] : (t & 6) == 4 ? v[4] : v[6];
}
// the first t (1..7) of the eight bytes lo | hi << 32 to p, at any address
struct __attribute__((packed, aligned(1))) Byte4Any { uint32_t x; };
struct __attribute__((packed, aligned(1))) Byte2Any { uint16_t x; };
__device__ __forceinline__ void store_byte8_head_any(int8_t* p, int t, uint32_t lo, uint32_t hi) {
    if (t & 4) *reinterpret_cast<Byte4Any*>(p) = Byte4Any{lo};
    const uint32_t rest = (t & 4) ? hi : lo;
    if (t & 2) *reinterpret_cast<Byte2Any*>(p + (t & 4)) = Byte2Any{(uint16_t)rest};
    if (t & 1) p[t & 6] = (int8_t)((t & 2) ? rest >> 16 : rest);
}

constexpr int kWave = 64;

__host__ __device__ inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// A null buffer with work to do would be a memory fault on the device, which ends the process: the
// launchers refuse it on the host (CPMK_EBADARG) once they know that the call is not empty.
template <class... P>
inline bool any_null(const P*... p) { return (... || (p == nullptr)); }

// Workgroups along a grid's x dimension: the runtime takes at most 2^31 - 1.
inline bool grid_fits(int64_t blocks) { return blocks <= 0x7fffffffll; }

// ---- wave64 reductions (butterfly over all 6 lane bits) -----------------------------
__device__ inline float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
    return v;
}
__device__ inline float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}
__device__ inline int32_t wave_sum_i32(int32_t v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}

// Sum over the wave with data-parallel-primitive operands instead of cross-lane reads through the LDS crossbar:
// six additions whose second operand comes from another lane (quad swaps, mirrors within 8 and 16 lanes, then the
// last lane of a row of 16 broadcast to the next row, and lane 31 to the upper half).  The total is in LANE 63 only.
__device__ inline int32_t wave_sum_i32_to_lane63(int32_t v) {
    v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xf, 0xf, true);      // quad_perm [1,0,3,2]
    v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xf, 0xf, true);      // quad_perm [2,3,0,1]
    v += __builtin_amdgcn_update_dpp(0, v, 0x141, 0xf, 0xf, true);     // row_half_mirror
    v += __builtin_amdgcn_update_dpp(0, v, 0x140, 0xf, 0xf, true);     // row_mirror
    v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);    // row_bcast15 into rows 1 and 3
    v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);    // row_bcast31 into rows 2 and 3
    return v;
}

// The same for an unsigned maximum, handed to every lane (as a wave-uniform value).
__device__ inline uint32_t wave_max_u32_uniform(uint32_t v) {
    v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xf, 0xf, true));
    v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xf, 0xf, true));
    v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x141, 0xf, 0xf, true));
    v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x140, 0xf, 0xf, true));
    v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xa, 0xf, false));
    v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xc, 0xf, false));
    return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}

// Block-wide reductions for blocks of NWAVES*64 threads.  `red` is LDS scratch of at least
// NWAVES floats.  Every thread returns the reduced value.  Contains two barriers so the
// scratch can be reused by the next call.
template <int NWAVES>
__device__ inline float block_max(float v, float* red) {
    v = wave_max(v);
    if (NWAVES == 1) return v;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    if (lane == 0) red[w] = v;
    __syncthreads();
    float r = red[0];
#pragma unroll
    for (int i = 1; i < NWAVES; ++i) r = fmaxf(r, red[i]);
    __syncthreads();
    return r;
}
template <int NWAVES>
__device__ inline float block_sum(float v, float* red) {
    v = wave_sum(v);
    if (NWAVES == 1) return v;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    if (lane == 0) red[w] = v;
    __syncthreads();
    float r = red[0];
#pragma unroll
    for (int i = 1; i < NWAVES; ++i) r += red[i];
    __syncthreads();
    return r;
}

// ---- |x| maxima on packed halves ---------------------------------------------------------
// Magnitudes of fp16 numbers that are not NaN order like their bit patterns with the sign cleared,
// so a running maximum needs one AND and one packed 16-bit integer maximum per two elements.  A NaN
// element has the largest patterns of all (above 0x7c00, infinity): a result above 0x7c00 says that
// the data held one, and the caller repeats the maximum in floating point, which skips NaN elements
// like the reference's fmaxf (cuda/gemm.cu:68-72).
typedef uint16_t ushort8_t __attribute__((ext_vector_type(8)));
__device__ inline ushort8_t absbits_max(ushort8_t m, half8_t x) {
    const uint4_t b = __builtin_bit_cast(uint4_t, x) & 0x7fff7fffu;
    return __builtin_elementwise_max(m, __builtin_bit_cast(ushort8_t, b));
}
__device__ inline uint32_t absbits_max_of(ushort8_t m) {
    uint32_t r = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) r = max(r, (uint32_t)m[e]);
    return r;
}
__device__ inline uint32_t wave_max_u32(uint32_t v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = max(v, (uint32_t)__shfl_xor((int)v, o, kWave));
    return v;
}

// ---- quantisation arithmetic ---------------------------------------------------------
// absmax/127 rounded to fp16.  The reference divides in double and converts
// double->float->half (cuda/gemm.cu:74); for every fp16 magnitude that equals the
// correctly rounded fp32 divide used here (checked exhaustively by the CPU tests).
__device__ inline half_t scale_from_absmax(float mx) { return (half_t)(mx / 127.0f); }

// int8( rint( x / s ) ): IEEE fp32 divide, round-half-even (cuda/gemm.cu:16).  Values that do
// not fit int8 (reachable only with a subnormal fp16 scale) saturate and NaN (0/0 for an
// all-zero row) gives 0; the reference's float->int8_t cast is undefined behaviour there.
__device__ inline int32_t quant_i8(float x, float s) {
    const float d = x / s;
    float q = __builtin_rintf(d);
    q = fminf(fmaxf(q, -128.0f), 127.0f);   // fmaxf/fminf drop a NaN operand ...
    return (d != d) ? 0 : (int32_t)q;       // ... so map NaN to 0 explicitly
}

// The same result from the row's reciprocal y = 1/s (one IEEE divide per row instead of one per
// element): a residual step restores the quotient closely enough that rint() lands on the same
// integer, ties included; when the residual is not finite (infinite operands, zero scale) the
// plain product already has the sign and size the divide would give.  Equality with quant_i8
// holds for every (fp16 value, fp16 scale) pair; tests/native/recip_round_check.c proves it by
// enumeration.
__device__ inline int32_t quant_i8_rcp(float x, float s, float y) {
    const float q0 = x * y;
    const float r = __builtin_fmaf(-s, q0, x);
    const float q1 = __builtin_fmaf(r, y, q0);
    const float d = __builtin_amdgcn_classf(r, 0x1f8) ? q1 : q0;      // 0x1f8: zero, subnormal or normal
    int32_t n;
    // v_cvt_i32_f32 saturates to the int32 range and turns NaN into 0
    asm("v_cvt_i32_f32 %0, %1" : "=v"(n) : "v"(__builtin_rintf(d)));
    return min(max(n, -128), 127);
}

// The short form for a scale that comes from the data it divides and is a normal fp16 number:
//     s = fp16(absmax / 127),  |x| <= absmax   =>   |x / s| <= 127 * (1 + 2^-11),
// so nothing saturates and the residual is always finite.  q + 1.5 * 2^23 lands in [2^23, 2^24),
// where the fp32 grid is the integers: the one round-to-nearest-even of that addition is rint(q), and
// the low byte of the sum's bit pattern is the two's-complement int8.  A NaN element (which the
// absmax ignores) propagates as a quiet NaN whose low byte is 0, the value the long form gives it.
// Equality with quant_i8 for every such (absmax, x) pair is proven by enumeration in
// tests/native/fused_round_check.c.  Returns the fp32 bit pattern; its low byte is the result.
__device__ inline bool scale_is_normal(half_t sh) {
    const uint16_t b = __builtin_bit_cast(uint16_t, sh);
    return b >= 0x0400u && b <= 0x7bffu;
}
__device__ inline uint32_t quant_i8_own_scale_bits(float x, float s, float y) {
    const float q0 = __builtin_fmaf(x, y, 0.0f);     // x * y (the sign of a zero does not matter below); as an fma the fp16 -> fp32 conversion of x folds into the instruction
    const float r = __builtin_fmaf(-s, q0, x);
    const float q1 = __builtin_fmaf(r, y, q0);
    float t = q1 + 12582912.0f;
    asm("" : "+v"(t));          // the sum must exist as a rounded fp32 number
    return __builtin_bit_cast(uint32_t, t);
}

// Low bytes of four integers (each already within int8 range) into one dword: three byte
// permutes.  v_perm_b32 selector bytes 0-3 pick from the second operand, 4-7 from the first, 0x0c is zero.
__device__ inline uint32_t pack4_i8(int32_t a, int32_t b, int32_t c, int32_t d) {
    const uint32_t lo = __builtin_amdgcn_perm((uint32_t)b, (uint32_t)a, 0x0c0c0400u);     // a | b << 8
    const uint32_t hi = __builtin_amdgcn_perm((uint32_t)d, (uint32_t)c, 0x0c0c0400u);     // c | d << 8
    return __builtin_amdgcn_perm(hi, lo, 0x05040100u);                                    // lo | hi << 16
}

// fp32 -> fp16 of a value that must first exist as a rounded fp32 number.  Without the
// register barrier the compiler folds "convert(multiply)" into v_fma_mixlo_f16, which rounds
// the exact product once, straight to fp16; the reference rounds to fp32 and then to fp16
// (cuda/gemm.cu:55), and the two differ on about one product in 10^4.
__device__ inline half_t round_f16(float v) {
    asm("" : "+v"(v));
    return (half_t)v;
}

// dequantising epilogue of cu_gemm_scale (cuda/gemm.cu:55): two fp32 multiplies in this order.
__device__ inline half_t dequant(int32_t acc, float sx, float sy) {
    return round_f16(((float)acc * sx) * sy);
}

// ---- host-side launch helpers ----------------------------------------------------------
// hipGetLastError() is sticky per host thread: an error left behind by an unrelated runtime
// call (for instance a failed device probe of another library) would otherwise be reported
// by the first launcher that asks.  Every launcher therefore clears it on entry.
inline void clear_stale_error() { (void)hipGetLastError(); }
// CPMK_ETIMEOUT if a kernel of an earlier launch on the current device gave up a bounded wait for another
// workgroup (it left NaN, or 0 in an int8 output, behind) and cpmk_async_status() has not taken the report
// yet, else 0: one load from pinned host memory that the kernel writes to (exchange.hip).
int async_failure();
// What every launcher returns after its launch: the runtime's error if the launch failed, else the pending
// asynchronous failure of an earlier kernel -- reported by the next call, like the runtime's own
// asynchronous errors (the reference raises them from its status checks, library/cudart.py:325-327).
inline int launch_status() {
    const int e = (int)hipGetLastError();
    return e != 0 ? e : async_failure();
}

// Map a linear workgroup index so that consecutive logical tiles land on the same XCD.
// Workgroups are dealt round-robin to the 8 XCDs of an MI355X (workgroup i -> XCD (i + k) % 8, k the same for a whole launch),
// each XCD has its own L2; tiles that share cache lines should therefore share an XCD.
__device__ inline uint32_t xcd_remap(uint32_t bid, uint32_t nblocks) {
    constexpr uint32_t kXcd = 8;
    const uint32_t per = nblocks / kXcd;          // tiles per XCD in the remappable part
    const uint32_t lim = per * kXcd;
    if (bid >= lim) return bid;                   // ragged tail keeps its index
    return (bid % kXcd) * per + bid / kXcd;
}

// 16 bytes per lane from global memory straight into LDS.  The LDS address is m0 + lane*16,
// so one wave instruction fills 1 KB of contiguous LDS; the swizzle is applied by choosing
// which global chunk each lane fetches.  Inline asm because the compiler would otherwise
// guard every later LDS read with vmcnt(0), which serialises the prefetch.
__device__ __forceinline__ void lds_dma16(uint32_t voff, const int8_t* sbase, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "s"(lds_addr)
                 : "memory");
}
// The same with the non-temporal hint: for data that is read once.
__device__ __forceinline__ void lds_dma16_nt(uint32_t voff, const int8_t* sbase, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1 nt" ::"v"(voff), "s"(sbase), "s"(lds_addr)
                 : "memory");
}
// s_waitcnt vmcnt(N) only (gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] << 14)
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// fp16 broadcast-matrix GEMV on the MFMA kernel of gemv_i8.hip (0, a HIP error code, or -1: shape not eligible)
int gemv_f16_coalesced(int32_t batch, int32_t dim_out, int32_t dim_in, const void* mat, const void* vec, void* out, hipStream_t st);
int gemv_f16_mfma(int32_t batch, int32_t dim_out, int32_t dim_in, const void* mat, const void* vec, void* out, hipStream_t st);

// Column scales (cu_gemm_calc_scale_transpose) on the register-tile team kernel of train.hip: 0, an error code, or -1 (shape not taken)
int col_absmax_team(int32_t batch, int32_t n, int32_t m, const void* mat, void* out, void* stream);

// Compute units of the current device (cached per device ordinal; 256 if the query fails).  The cache
// is atomic: host threads that make their first call together each ask the runtime and store the
// same value.
inline int compute_units() {
    static std::atomic<int> cus[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    int n = cus[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cus[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

// Dynamic LDS above the default limit must be enabled per kernel and device.  `done` is the
// kernel's array of 64 per-device flags (static storage, so zero at start); the attribute call is
// idempotent, so host threads racing through their first launch at worst all make it.
inline int enable_dynamic_lds(const void* kern, int bytes, std::atomic<bool>* done) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    if (done[dev].load(std::memory_order_acquire)) return 0;
    const hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) return (int)e;
    done[dev].store(true, std::memory_order_release);
    return 0;
}

}  // namespace cpmk
