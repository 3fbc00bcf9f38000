// What the chip sustains, measured with kernels that do nothing else: the yardsticks bench.py's
// `--only ceilings` leg reports beside the library's own kernels.  Built into its own shared
// library (libcpmk_ceilings.so); nothing here is linked into or called by libcpmk_hip.so.
//
//   ceil_mfma_i8        v_mfma_i32_32x32x32_i8 back to back from registers, no memory traffic in the
//                       loop: 8 waves per workgroup, 8 accumulator tiles per wave and two sets of
//                       operand fragments used in turn -- the register shape of the library's
//                       256x256 GEMM tile -- so the result is the matrix pipe's rate on the given
//                       operand bytes (all zero: the clock stays high; random: it drops)
//   ceil_mfma_i8_16x16x64   the same wave tile with v_mfma_i32_16x16x64_i8
//   ceil_read / ceil_write / ceil_copy      contiguous 16-byte accesses; `nontemporal` != 0 gives the loads and
//                       stores the non-temporal hint (data touched once), which a 1 GiB copy rewards with 10 %
//   ceil_copy_segments_persistent   the same tiles through one persistent workgroup per compute unit that loads the next
//                       tile while it stores the current one and takes its tiles from a counter: what the many-tile
//                       softmax's structure reaches without its arithmetic
//   ceil_read_span      256 workgroups read one contiguous share each, every load requested at once, and stamp
//                       their start and end with the 100 MHz wall clock: last end - first start is the time the
//                       memory system needs for those bytes, without what a kernel launch costs around it
//   ceil_empty          a kernel that does nothing: what one launch costs between two others
//   ceil_xcc_ids        which XCD each workgroup of a launch runs on
//   ceil_read_gemv_pattern  a decode GEMV's loads with the matrix straight in the MFMA operand layout (and the vectors every workgroup reads), no arithmetic
//   ceil_copy_segments  a (rows, row_bytes) matrix copied in tiles of `seg` bytes x many rows, one
//                       tile per 1024-thread workgroup, all loads of a tile before its stores: the
//                       access pattern of the dim-1 kernels (layernorm, softmax) without arithmetic
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef int int4_t __attribute__((ext_vector_type(4)));
typedef int int16_tv __attribute__((ext_vector_type(16)));

namespace {

__global__ __launch_bounds__(512) void k_mfma_i8(const int4_t* __restrict__ operands, int32_t iters, int32_t* sink) {
    // 12 fragments per lane: two sets of 4 row-operand and 2 column-operand fragments
    int4_t fp[2][4], fq[2][2];
    const int t = threadIdx.x;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
#pragma unroll
        for (int i = 0; i < 4; ++i) fp[s][i] = operands[(size_t)(s * 6 + i) * 512 + t];
#pragma unroll
        for (int j = 0; j < 2; ++j) fq[s][j] = operands[(size_t)(s * 6 + 4 + j) * 512 + t];
    }
    int16_tv acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;
    for (int32_t it = 0; it < iters; ++it) {
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fq[s][j], fp[s][i], acc[i][j], 0, 0, 0);
    }
    int32_t x = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) x ^= acc[i][j][e];
    if (x == 0x5a5a5a5a) sink[0] = x;       // keeps the loop alive; practically never true
}

// The same amount of work per wave with v_mfma_i32_16x16x64_i8: a 128x64 wave tile is 8 x 4 tiles of
// 16x16 (128 accumulator registers, as above), a k-step of 64 bytes takes 8 + 4 operand fragments.
__global__ __launch_bounds__(512) void k_mfma_i8_16(const int4_t* __restrict__ operands, int32_t iters, int32_t* sink) {
    int4_t fp[8], fq[4];
    const int t = threadIdx.x;
#pragma unroll
    for (int i = 0; i < 8; ++i) fp[i] = operands[(size_t)i * 512 + t];
#pragma unroll
    for (int j = 0; j < 4; ++j) fq[j] = operands[(size_t)(8 + j) * 512 + t];
    int4_t acc[8][4];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = int4_t{0, 0, 0, 0};
    for (int32_t it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fq[j], fp[i], acc[i][j], 0, 0, 0);
    }
    int32_t x = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) x ^= acc[i][j].x ^ acc[i][j].y ^ acc[i][j].z ^ acc[i][j].w;
    if (x == 0x5a5a5a5a) sink[0] = x;
}

template <bool NTEMP>
__global__ __launch_bounds__(256) void k_read(const int4_t* __restrict__ p, int64_t n16, int4_t* sink) {
    int64_t i = (int64_t)blockIdx.x * 1024 + threadIdx.x;
    int4_t a = {0, 0, 0, 0};
#pragma unroll
    for (int u = 0; u < 4; ++u)
        if (i + u * 256 < n16) a += NTEMP ? __builtin_nontemporal_load(p + i + u * 256) : p[i + u * 256];
    if (a.x == 0x12345678 && a.y == 1) sink[0] = a;
}

__global__ void k_empty(int4_t* sink) {
    if (threadIdx.x == 0x7fffffff) sink[0] = int4_t{1, 2, 3, 4};      // never
}

// out[b] = the XCC (XCD) that workgroup b of the launch runs on, as the hardware register says
__global__ void k_xcc_ids(int32_t* out) {
    uint32_t xcc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    if (threadIdx.x == 0) out[blockIdx.x] = (int32_t)(xcc & 15u);
}

// 512 threads, NLD pieces of 16 bytes per thread: a share of NLD * 8 KB per workgroup; stamps[2b], [2b+1] = start, end of workgroup b
template <int NLD>
__global__ __launch_bounds__(512) void k_read_span(const char* __restrict__ src, int4_t* sink, unsigned long long* stamps) {
    const unsigned long long t0 = wall_clock64();
    const char* base = src + (int64_t)blockIdx.x * (NLD * 8192) + threadIdx.x * 16;
    int4_t v[NLD];
#pragma unroll
    for (int i = 0; i < NLD; ++i) v[i] = __builtin_nontemporal_load(reinterpret_cast<const int4_t*>(base + i * 8192));
    int4_t a = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < NLD; ++i) a += v[i];
    if (a.x == 0x12345678 && a.y == 1) sink[0] = a;
    __syncthreads();
    if (threadIdx.x == 0) {
        stamps[2 * blockIdx.x] = t0;
        stamps[2 * blockIdx.x + 1] = wall_clock64();
    }
}

// The memory traffic of a decode GEMV that loads its matrix straight in the MFMA operand layout (the library's kernel
// does not: it reads 4 rows x 256 bytes per instruction), without the arithmetic: 40 rows of 4096 bytes per workgroup, wave w bytes
// [512w, 512w + 512) of every row, lane (r, q) 16 bytes of row 16g + r -- the MFMA operand layout, in which an
// instruction touches 64 bytes of 16 rows -- and, if VEC, the 128 KB every workgroup reads alike (32 vectors),
// requested behind the first 16 rows.  NTL: non-temporal matrix loads.  Stamps as k_read_span.
template <int VEC, int NTL>
__global__ __launch_bounds__(512) void k_read_gemv_pattern(const char* __restrict__ mat, const char* __restrict__ vec, int4_t* sink,
                                                           unsigned long long* stamps) {
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, r = lane & 15, q = lane >> 4;
    const unsigned long long t0 = wall_clock64();
    const int row0 = blockIdx.x * 40;
    int4_t v[3][8], u[VEC ? 16 : 1];
    auto rows = [&](int g) __attribute__((always_inline)) {
        const int row = row0 + min(g * 16 + r, 39);
        const char* rp = mat + (uint32_t)row * 4096u + w * 512 + q * 16;
#pragma unroll
        for (int kb = 0; kb < 8; ++kb)
            v[g][kb] = NTL ? __builtin_nontemporal_load(reinterpret_cast<const int4_t*>(rp + kb * 64)) : *reinterpret_cast<const int4_t*>(rp + kb * 64);
    };
    rows(0);
    if (VEC) {
#pragma unroll
        for (int i = 0; i < 16; ++i) u[i] = *reinterpret_cast<const int4_t*>(vec + ((int64_t)i * 512 + tid) * 16);
    }
    rows(1);
    rows(2);
    int4_t a = {0, 0, 0, 0};
#pragma unroll
    for (int g = 0; g < 3; ++g)
#pragma unroll
        for (int kb = 0; kb < 8; ++kb) a += v[g][kb];
    if (VEC) {
#pragma unroll
        for (int i = 0; i < 16; ++i) a += u[i];
    }
    if (a.x == 0x12345678 && a.y == 1) sink[0] = a;
    __syncthreads();
    if (threadIdx.x == 0) {
        stamps[2 * blockIdx.x] = t0;
        stamps[2 * blockIdx.x + 1] = wall_clock64();
    }
}

__global__ __launch_bounds__(256) void k_write(int4_t* p, int64_t n16) {
    int64_t i = (int64_t)blockIdx.x * 1024 + threadIdx.x;
    const int4_t v = {1, 2, 3, (int)threadIdx.x};
#pragma unroll
    for (int u = 0; u < 4; ++u)
        if (i + u * 256 < n16) p[i + u * 256] = v;
}

template <bool NTEMP>
__global__ __launch_bounds__(256) void k_copy(const int4_t* __restrict__ p, int4_t* __restrict__ q, int64_t n16) {
    int64_t i = (int64_t)blockIdx.x * 1024 + threadIdx.x;
    int4_t v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
        if (i + u * 256 < n16) v[u] = NTEMP ? __builtin_nontemporal_load(p + i + u * 256) : p[i + u * 256];
#pragma unroll
    for (int u = 0; u < 4; ++u)
        if (i + u * 256 < n16) {
            if (NTEMP) __builtin_nontemporal_store(v[u], q + i + u * 256);
            else q[i + u * 256] = v[u];
        }
}

// Tile = TROWS rows x seg bytes; a workgroup of 1024 threads holds it in 8 x 16 bytes per thread.
template <bool NTEMP>
__global__ __launch_bounds__(1024) void k_copy_segments(const char* __restrict__ src, char* __restrict__ dst, int32_t row_bytes,
                                                        int32_t seg, int32_t tiles_per_row, int32_t tile_rows) {
    const int ppr = seg / 16;                    // 16-byte pieces per row segment
    const int rpp = 1024 / ppr;                  // rows per pass of the workgroup
    const int64_t tr = blockIdx.x / tiles_per_row, tc = blockIdx.x % tiles_per_row;
    const int64_t base = tr * (int64_t)tile_rows * row_bytes + tc * seg + (threadIdx.x % ppr) * 16;
    const int r0 = threadIdx.x / ppr;
    int4_t v[8];
#pragma unroll
    for (int p = 0; p < 8; ++p) {
        const int4_t* s = reinterpret_cast<const int4_t*>(src + base + (int64_t)(r0 + p * rpp) * row_bytes);
        v[p] = NTEMP ? __builtin_nontemporal_load(s) : *s;
    }
#pragma unroll
    for (int p = 0; p < 8; ++p) {
        int4_t* d = reinterpret_cast<int4_t*>(dst + base + (int64_t)(r0 + p * rpp) * row_bytes);
        if (NTEMP) __builtin_nontemporal_store(v[p], d);
        else *d = v[p];
    }
}

// The same tiles copied by persistent workgroups (one per compute unit) that load the next tile while they store the
// current one and take their tiles from a counter in device memory: the shape of the library's many-tile softmax.
// sched[0] = tiles handed out beyond the first round, sched[1] = workgroups done (the last one clears both).
template <int LPR>
__global__ __launch_bounds__(1024) void k_copy_segments_persistent(const char* __restrict__ src, char* __restrict__ dst, int32_t row_bytes,
                                                                   uint32_t ntiles, unsigned int* sched) {
    constexpr int SEG = LPR * 16, RPP = 1024 / LPR, ROWS = RPP * 8;
    __shared__ uint32_t s_next;
    const int tid = threadIdx.x, cg = tid % LPR, rg = tid / LPR;
    const uint32_t tpr = (uint32_t)row_bytes / SEG;
    auto addr = [&](uint32_t t, int p) -> int64_t {
        const int64_t tr = t / tpr, tc = t % tpr;
        return (tr * ROWS + p * RPP + rg) * row_bytes + tc * SEG + cg * 16;
    };
    uint32_t t = blockIdx.x;
    int4_t v[8], w[8];
#pragma unroll
    for (int p = 0; p < 8; ++p) v[p] = __builtin_nontemporal_load(reinterpret_cast<const int4_t*>(src + addr(t, p)));
    if (tid == 0) s_next = gridDim.x + atomicAdd(&sched[0], 1u);
    __syncthreads();
    uint32_t tn = s_next;
    while (t < ntiles) {
        if (tn < ntiles) {
#pragma unroll
            for (int p = 0; p < 8; ++p) w[p] = __builtin_nontemporal_load(reinterpret_cast<const int4_t*>(src + addr(tn, p)));
        }
        __syncthreads();
        if (tid == 0) s_next = gridDim.x + atomicAdd(&sched[0], 1u);
        __syncthreads();
        const uint32_t tnn = s_next;
#pragma unroll
        for (int p = 0; p < 8; ++p) __builtin_nontemporal_store(v[p], reinterpret_cast<int4_t*>(dst + addr(t, p)));
#pragma unroll
        for (int p = 0; p < 8; ++p) v[p] = w[p];
        t = tn;
        tn = tnn;
    }
    if (tid == 0 && atomicAdd(&sched[1], 1u) == gridDim.x - 1) {
        atomicExch(&sched[0], 0u);
        atomicExch(&sched[1], 0u);
    }
}

int status() { return (int)hipGetLastError(); }

}  // namespace

extern "C" {

// operands: 12 * 512 * 16 = 98304 bytes.  One workgroup per compute unit is the caller's choice of `workgroups`;
// `waves` per workgroup: 8 = two per SIMD (the GEMM's occupancy), 4 = one per SIMD.
// int8 operations done: workgroups * waves * iters * 16 MFMAs * 2 * 32^3.
int ceil_mfma_i8(const void* operands, int32_t workgroups, int32_t waves, int32_t iters, void* sink, void* stream) {
    if (workgroups < 1 || iters < 0 || waves < 1 || waves > 8) return 1;
    hipLaunchKernelGGL(k_mfma_i8, dim3((unsigned)workgroups), dim3((unsigned)waves * 64), 0, (hipStream_t)stream,
                       (const int4_t*)operands, iters, (int32_t*)sink);
    return status();
}

// The 16x16x64 form of the same instruction: int8 operations done = workgroups * waves * iters * 32 MFMAs * 2 * 16*16*64.
int ceil_mfma_i8_16x16x64(const void* operands, int32_t workgroups, int32_t waves, int32_t iters, void* sink, void* stream) {
    if (workgroups < 1 || iters < 0 || waves < 1 || waves > 8) return 1;
    hipLaunchKernelGGL(k_mfma_i8_16, dim3((unsigned)workgroups), dim3((unsigned)waves * 64), 0, (hipStream_t)stream,
                       (const int4_t*)operands, iters, (int32_t*)sink);
    return status();
}

int ceil_read(const void* src, int64_t bytes, void* sink, int nontemporal, void* stream) {
    const int64_t n16 = bytes / 16;
    const dim3 grid((unsigned)((n16 + 1023) / 1024));
    if (nontemporal) hipLaunchKernelGGL(k_read<true>, grid, dim3(256), 0, (hipStream_t)stream, (const int4_t*)src, n16, (int4_t*)sink);
    else hipLaunchKernelGGL(k_read<false>, grid, dim3(256), 0, (hipStream_t)stream, (const int4_t*)src, n16, (int4_t*)sink);
    return status();
}

// `workgroups` x 20 x 8192 bytes from src, one contiguous share per workgroup; stamps: 2 x workgroups 64-bit words (100 MHz ticks)
int ceil_read_span(const void* src, int32_t workgroups, void* sink, void* stamps, void* stream) {
    if (workgroups < 1) return 1;
    hipLaunchKernelGGL(k_read_span<20>, dim3((unsigned)workgroups), dim3(512), 0, (hipStream_t)stream, (const char*)src, (int4_t*)sink,
                       (unsigned long long*)stamps);
    return status();
}

// the XCD of each of `workgroups` workgroups of one launch (int32 each)
int ceil_xcc_ids(void* out, int32_t workgroups, int32_t threads, void* stream) {
    if (workgroups < 1 || threads < 1 || threads > 1024) return 1;
    hipLaunchKernelGGL(k_xcc_ids, dim3((unsigned)workgroups), dim3((unsigned)threads), 0, (hipStream_t)stream, (int32_t*)out);
    return status();
}

// 256 workgroups x 40 rows of 4096 bytes from src in the GEMV's access pattern; vec: 128 KB that every workgroup reads (or null)
int ceil_read_gemv_pattern(const void* src, const void* vec, int nontemporal, void* sink, void* stamps, void* stream) {
    const dim3 g(256), b(512);
    hipStream_t st = (hipStream_t)stream;
    if (vec != nullptr) {
        if (nontemporal) hipLaunchKernelGGL((k_read_gemv_pattern<1, 1>), g, b, 0, st, (const char*)src, (const char*)vec, (int4_t*)sink, (unsigned long long*)stamps);
        else hipLaunchKernelGGL((k_read_gemv_pattern<1, 0>), g, b, 0, st, (const char*)src, (const char*)vec, (int4_t*)sink, (unsigned long long*)stamps);
    } else {
        if (nontemporal) hipLaunchKernelGGL((k_read_gemv_pattern<0, 1>), g, b, 0, st, (const char*)src, (const char*)vec, (int4_t*)sink, (unsigned long long*)stamps);
        else hipLaunchKernelGGL((k_read_gemv_pattern<0, 0>), g, b, 0, st, (const char*)src, (const char*)vec, (int4_t*)sink, (unsigned long long*)stamps);
    }
    return status();
}

int ceil_empty(int32_t workgroups, int32_t threads, void* sink, void* stream) {
    if (workgroups < 1 || threads < 1 || threads > 1024) return 1;
    hipLaunchKernelGGL(k_empty, dim3((unsigned)workgroups), dim3((unsigned)threads), 0, (hipStream_t)stream, (int4_t*)sink);
    return status();
}

int ceil_write(void* dst, int64_t bytes, void* stream) {
    const int64_t n16 = bytes / 16;
    hipLaunchKernelGGL(k_write, dim3((unsigned)((n16 + 1023) / 1024)), dim3(256), 0, (hipStream_t)stream, (int4_t*)dst, n16);
    return status();
}

int ceil_copy(const void* src, void* dst, int64_t bytes, int nontemporal, void* stream) {
    const int64_t n16 = bytes / 16;
    const dim3 grid((unsigned)((n16 + 1023) / 1024));
    if (nontemporal) hipLaunchKernelGGL(k_copy<true>, grid, dim3(256), 0, (hipStream_t)stream, (const int4_t*)src, (int4_t*)dst, n16);
    else hipLaunchKernelGGL(k_copy<false>, grid, dim3(256), 0, (hipStream_t)stream, (const int4_t*)src, (int4_t*)dst, n16);
    return status();
}

// rows x row_bytes matrix; seg in {32, 64, 128, 256, 512, 1024} must divide row_bytes; a tile is
// 131072 / seg rows, which must divide rows.
int ceil_copy_segments(const void* src, void* dst, int64_t rows, int32_t row_bytes, int32_t seg, int nontemporal, void* stream) {
    if (seg < 32 || seg > 1024 || (seg & (seg - 1)) || row_bytes % seg) return 1;
    const int32_t tile_rows = 131072 / seg;
    if (rows % tile_rows) return 1;
    const int64_t tiles = rows / tile_rows * (row_bytes / seg);
    if (tiles > 0x7fffffff) return 1;
    if (nontemporal)
        hipLaunchKernelGGL(k_copy_segments<true>, dim3((unsigned)tiles), dim3(1024), 0, (hipStream_t)stream, (const char*)src, (char*)dst,
                           row_bytes, seg, row_bytes / seg, tile_rows);
    else
        hipLaunchKernelGGL(k_copy_segments<false>, dim3((unsigned)tiles), dim3(1024), 0, (hipStream_t)stream, (const char*)src, (char*)dst,
                           row_bytes, seg, row_bytes / seg, tile_rows);
    return status();
}

// The persistent form: `workgroups` workgroups (at most the number of tiles); seg in {128, 256, 512}; sched: two zeroed 32-bit words
// that the kernel leaves zeroed.  rows must be a multiple of the tile's 131072 / seg rows.
int ceil_copy_segments_persistent(const void* src, void* dst, int64_t rows, int32_t row_bytes, int32_t seg, int32_t workgroups, void* sched,
                                  void* stream) {
    if ((seg != 128 && seg != 256 && seg != 512) || row_bytes % seg) return 1;
    const int32_t tile_rows = 131072 / seg;
    if (rows % tile_rows) return 1;
    const int64_t tiles = rows / tile_rows * (row_bytes / seg);
    if (tiles > 0x7fffffff || workgroups < 1 || workgroups > tiles) return 1;
    const dim3 grid((unsigned)workgroups);
    if (seg == 128)
        hipLaunchKernelGGL(k_copy_segments_persistent<8>, grid, dim3(1024), 0, (hipStream_t)stream, (const char*)src, (char*)dst, row_bytes,
                           (uint32_t)tiles, (unsigned int*)sched);
    else if (seg == 256)
        hipLaunchKernelGGL(k_copy_segments_persistent<16>, grid, dim3(1024), 0, (hipStream_t)stream, (const char*)src, (char*)dst, row_bytes,
                           (uint32_t)tiles, (unsigned int*)sched);
    else
        hipLaunchKernelGGL(k_copy_segments_persistent<32>, grid, dim3(1024), 0, (hipStream_t)stream, (const char*)src, (char*)dst, row_bytes,
                           (uint32_t)tiles, (unsigned int*)sched);
    return status();
}

}  // extern "C"
