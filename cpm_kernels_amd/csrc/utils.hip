// Small utilities of the reference's kernels layer: transpose (cuda/transpose.cu:6-24) and the
// generation helpers of cuda/utils.cu:31-101 (array_add, adjustify_logits, copy_extend_buffer,
// has_nan_inf, copy_pos_hidden).
#include "common.h"

namespace cpmk {

// (batch, n, m) -> (batch, m, n) through a 64x64 LDS tile.  IN / OUT: eight halves per global load / store where a
// piece of eight lies inside its row (a 16-byte access at whatever address it starts: global accesses need no
// alignment), single halves for the piece across a row's end; the scalar form (IN = OUT = false) for rows under eight.
template <bool IN, bool OUT>
__global__ __launch_bounds__(256) void k_transpose(int32_t n, int32_t m, const half_t* __restrict__ in, half_t* __restrict__ out) {
    __shared__ __attribute__((aligned(16))) half_t tile[64][72];    // pitch 144 bytes: 16-byte aligned rows, odd multiple of 16 bytes
    const int64_t boff = (int64_t)blockIdx.z * n * m;
    const int32_t r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
    const int pc = threadIdx.x & 7, rr = threadIdx.x >> 3;          // 8 pieces x 32 rows per pass
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    if constexpr (IN) {
#pragma unroll
        for (int ps = 0; ps < 2; ++ps) {
            const int r = ps * 32 + rr;
            const int32_t c = c0 + pc * 8;
            if (r0 + r < n && c < m) {
                const half_t* src = in + boff + (int64_t)(r0 + r) * m + c;
                half8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
                if (c + 8 <= m) v = load_half8_any(src);
                else v = load_half8_head_any(src, m - c, v);
                *reinterpret_cast<half8_t*>(&tile[r][pc * 8]) = v;
            }
        }
    } else {
        for (int r = ty; r < 64; r += 4)
            if (r0 + r < n && c0 + tx < m) tile[r][tx] = in[boff + (int64_t)(r0 + r) * m + c0 + tx];
    }
    __syncthreads();
    if constexpr (OUT) {
#pragma unroll
        for (int ps = 0; ps < 2; ++ps) {
            const int c = ps * 32 + rr;                     // row of the transposed tile
            const int32_t r = r0 + pc * 8;
            if (c0 + c < m && r < n) {
                half8_t v;
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] = tile[pc * 8 + e][c];
                half_t* dst = out + boff + (int64_t)(c0 + c) * n + r;
                if (r + 8 <= n) store_half8_any(dst, v);
                else store_half8_head_any(dst, n - r, v);
            }
        }
    } else {
        for (int c = ty; c < 64; c += 4)
            if (c0 + c < m && r0 + tx < n) out[boff + (int64_t)(c0 + c) * n + r0 + tx] = tile[tx][c];
    }
}

// (batch, n, m) -> (batch, m, n) of bytes: 64x64 tile through LDS.  IN / OUT: sixteen bytes per global load / store where
// a piece of sixteen lies inside its row (at whatever address it starts: global accesses need no alignment), single
// bytes for the piece across a row's end; the scalar form (false) for rows under sixteen bytes.
struct __attribute__((packed, aligned(1))) Byte16Any { uint32_t x, y, z, w; };

template <bool IN, bool OUT>
__global__ __launch_bounds__(256) void k_transpose_i8(int32_t n, int32_t m, const int8_t* __restrict__ in, int8_t* __restrict__ out) {
    __shared__ __attribute__((aligned(16))) int8_t tile[64][68];        // pitch 68: dword-aligned rows, 17 banks apart
    const int64_t boff = (int64_t)blockIdx.z * n * m;
    const int32_t r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
    const int pc = threadIdx.x & 3, rr = threadIdx.x >> 2;          // 4 pieces of 16 bytes x 64 rows
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    if constexpr (IN) {
        const int32_t c = c0 + pc * 16;
        if (r0 + rr < n && c < m) {
            const int8_t* src = in + boff + (int64_t)(r0 + rr) * m + c;
            if (c + 16 <= m) {
                const Byte16Any v = *reinterpret_cast<const Byte16Any*>(src);
                uint32_t* dst = reinterpret_cast<uint32_t*>(&tile[rr][pc * 16]);
                dst[0] = v.x; dst[1] = v.y; dst[2] = v.z; dst[3] = v.w;
            } else {
                for (int e = 0; e < m - c; ++e) tile[rr][pc * 16 + e] = src[e];
            }
        }
    } else {
        for (int r = ty; r < 64; r += 4)
            if (r0 + r < n && c0 + tx < m) tile[r][tx] = in[boff + (int64_t)(r0 + r) * m + c0 + tx];
    }
    __syncthreads();
    if constexpr (OUT) {
        // row rr of the transposed tile = column rr of the tile; this thread's 16 bytes are its rows pc*16 .. pc*16+15
        const int32_t r = r0 + pc * 16;
        if (c0 + rr < m && r < n) {
            int8_t* dst = out + boff + (int64_t)(c0 + rr) * n + r;
            if (r + 16 <= n) {
                uint32_t w[4];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    uint32_t x = 0;
#pragma unroll
                    for (int e = 0; e < 4; ++e) x |= (uint32_t)(uint8_t)tile[pc * 16 + q * 4 + e][rr] << (8 * e);
                    w[q] = x;
                }
                *reinterpret_cast<Byte16Any*>(dst) = Byte16Any{w[0], w[1], w[2], w[3]};
            } else {
                for (int e = 0; e < n - r; ++e) dst[e] = tile[pc * 16 + e][rr];
            }
        }
    } else {
        for (int c = ty; c < 64; c += 4)
            if (c0 + c < m && r0 + tx < n) out[boff + (int64_t)(c0 + c) * n + r0 + tx] = tile[tx][c];
    }
}

__global__ void k_array_add(int32_t* arr, int32_t pos, int32_t val) {
    if (threadIdx.x == 0) arr[pos] += val;
}

__global__ __launch_bounds__(256) void k_adjustify_logits(int64_t total, half_t* logits, float temperature, float frequency_penalty,
                                                          float presence_penalty, const int32_t* __restrict__ frequency) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    float v = (float)logits[i];
    const int32_t freq = frequency[i];
    v /= temperature;
    v -= frequency_penalty * (float)freq;
    v -= presence_penalty * (freq > 0 ? 1.0f : 0.0f);
    logits[i] = round_f16(v);
}

__global__ __launch_bounds__(256) void k_copy_extend(int32_t old_size, int32_t nw_size, const half_t* __restrict__ old_buf,
                                                     half_t* __restrict__ nw_buf) {
    const int32_t col = blockIdx.x * 256 + threadIdx.x;
    if (col < old_size) nw_buf[(int64_t)blockIdx.y * nw_size + col] = old_buf[(int64_t)blockIdx.y * old_size + col];
}

// the same, 8 halves per thread (both row lengths multiples of 8, 16-byte aligned buffers)
__global__ __launch_bounds__(256) void k_copy_extend_wide(int32_t old_size, int32_t nw_size, const half_t* __restrict__ old_buf,
                                                          half_t* __restrict__ nw_buf) {
    const int32_t col = (blockIdx.x * 256 + threadIdx.x) * 8;
    if (col < old_size)
        *reinterpret_cast<half8_t*>(nw_buf + (int64_t)blockIdx.y * nw_size + col) =
            *reinterpret_cast<const half8_t*>(old_buf + (int64_t)blockIdx.y * old_size + col);
}

// out[0] = 1 when any element is +-inf or NaN; out is left untouched otherwise (the caller clears it).
__global__ __launch_bounds__(256) void k_has_nan_inf(int64_t n, const uint16_t* __restrict__ inp, int8_t* out) {
    bool bad = false;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256)
        bad |= (inp[i] & 0x7c00u) == 0x7c00u;       // exponent all ones: inf or NaN
    if (__ballot(bad) != 0 && (threadIdx.x & 63) == 0) out[0] = 1;
}

__global__ __launch_bounds__(256) void k_copy_pos_hidden(int32_t hidden_size, int32_t seq_len, int32_t pos,
                                                         const half_t* __restrict__ inp, half_t* __restrict__ out) {
    const int32_t col = blockIdx.x * 256 + threadIdx.x;
    if (col < hidden_size)
        out[(int64_t)blockIdx.y * hidden_size + col] = inp[((int64_t)blockIdx.y * hidden_size + col) * seq_len + pos];
}

}  // namespace cpmk

using namespace cpmk;

extern "C" {

int cpmk_transpose(int32_t batch, int32_t n, int32_t m, const void* inp, void* out, void* stream) {
    clear_stale_error();
    if (batch < 0 || n < 0 || m < 0) return CPMK_EBADARG;
    if ((int64_t)batch * n * m == 0) return 0;
    if (any_null(inp, out)) return CPMK_EBADARG;
    if (ceil_div(n, 64) > 65535) return CPMK_ETOOBIG;
    const bool win = m >= 8, wout = n >= 8;       // pieces of eight on a side whose rows hold at least one
    // the batch is the grid's z dimension (at most 65535): larger batches go out in several launches
    for (int64_t b0 = 0; b0 < batch; b0 += 65535) {
        const int64_t nb = batch - b0 < 65535 ? batch - b0 : 65535;
        const dim3 grid((unsigned)ceil_div(m, 64), (unsigned)ceil_div(n, 64), (unsigned)nb);
        const half_t* src = (const half_t*)inp + b0 * n * m;
        half_t* dst = (half_t*)out + b0 * n * m;
        auto go = [&](auto kern) { hipLaunchKernelGGL(kern, grid, dim3(256), 0, (hipStream_t)stream, n, m, src, dst); };
        if (win) { if (wout) go(k_transpose<true, true>); else go(k_transpose<true, false>); }
        else { if (wout) go(k_transpose<false, true>); else go(k_transpose<false, false>); }
        if (int e = launch_status()) return e;
    }
    return 0;
}

int cpmk_transpose_i8(int32_t batch, int32_t n, int32_t m, const void* inp, void* out, void* stream) {
    clear_stale_error();
    if (batch < 0 || n < 0 || m < 0) return CPMK_EBADARG;
    if ((int64_t)batch * n * m == 0) return 0;
    if (any_null(inp, out)) return CPMK_EBADARG;
    if (ceil_div(n, 64) > 65535) return CPMK_ETOOBIG;
    const bool win = m >= 16, wout = n >= 16;       // pieces of sixteen on a side whose rows hold at least one
    for (int64_t b0 = 0; b0 < batch; b0 += 65535) {       // (grid z: at most 65535 batch entries per launch)
        const int64_t nb = batch - b0 < 65535 ? batch - b0 : 65535;
        const dim3 grid((unsigned)ceil_div(m, 64), (unsigned)ceil_div(n, 64), (unsigned)nb);
        const int8_t* src = (const int8_t*)inp + b0 * n * m;
        int8_t* dst = (int8_t*)out + b0 * n * m;
        auto go = [&](auto kern) { hipLaunchKernelGGL(kern, grid, dim3(256), 0, (hipStream_t)stream, n, m, src, dst); };
        if (win) { if (wout) go(k_transpose_i8<true, true>); else go(k_transpose_i8<true, false>); }
        else { if (wout) go(k_transpose_i8<false, true>); else go(k_transpose_i8<false, false>); }
        if (int e = launch_status()) return e;
    }
    return 0;
}

int cpmk_array_add(void* array, int32_t pos, int32_t val, void* stream) {
    clear_stale_error();
    if (pos < 0 || !array) return CPMK_EBADARG;
    hipLaunchKernelGGL(k_array_add, dim3(1), dim3(64), 0, (hipStream_t)stream, (int32_t*)array, pos, val);
    return launch_status();
}

int cpmk_adjustify_logits(int32_t batch, int32_t n, void* logits, float temperature, float frequency_penalty, float presence_penalty,
                          const void* frequency, void* stream) {
    clear_stale_error();
    if (batch < 0 || n < 0) return CPMK_EBADARG;
    const int64_t total = (int64_t)batch * n;
    if (total == 0) return 0;
    if (any_null(logits, frequency)) return CPMK_EBADARG;
    hipLaunchKernelGGL(k_adjustify_logits, dim3((unsigned)ceil_div(total, 256)), dim3(256), 0, (hipStream_t)stream, total,
                       (half_t*)logits, temperature, frequency_penalty, presence_penalty, (const int32_t*)frequency);
    return launch_status();
}

int cpmk_copy_extend_buffer(int32_t batch, int32_t old_size, int32_t nw_size, const void* old_buffer, void* new_buffer, void* stream) {
    clear_stale_error();
    if (batch < 0 || old_size < 0 || nw_size < old_size) return CPMK_EBADARG;
    if ((int64_t)batch * old_size == 0) return 0;
    if (any_null(old_buffer, new_buffer)) return CPMK_EBADARG;
    const bool wide = old_size % 8 == 0 && nw_size % 8 == 0 && aligned16(old_buffer) && aligned16(new_buffer);
    for (int64_t b0 = 0; b0 < batch; b0 += 65535) {       // (grid y: at most 65535 batch entries per launch)
        const int64_t nb = batch - b0 < 65535 ? batch - b0 : 65535;
        const half_t* src = (const half_t*)old_buffer + b0 * old_size;
        half_t* dst = (half_t*)new_buffer + b0 * nw_size;
        if (wide)
            hipLaunchKernelGGL(k_copy_extend_wide, dim3((unsigned)ceil_div(old_size, 2048), (unsigned)nb), dim3(256), 0,
                               (hipStream_t)stream, old_size, nw_size, src, dst);
        else
            hipLaunchKernelGGL(k_copy_extend, dim3((unsigned)ceil_div(old_size, 256), (unsigned)nb), dim3(256), 0, (hipStream_t)stream,
                               old_size, nw_size, src, dst);
        if (int e = launch_status()) return e;
    }
    return 0;
}

int cpmk_has_nan_inf(int64_t n, const void* inp, void* out, void* stream) {
    clear_stale_error();
    if (n < 0) return CPMK_EBADARG;
    if (n == 0) return 0;
    if (any_null(inp, out)) return CPMK_EBADARG;
    const int64_t blocks = ceil_div(n, 256 * 16);
    hipLaunchKernelGGL(k_has_nan_inf, dim3((unsigned)(blocks > 2048 ? 2048 : blocks)), dim3(256), 0, (hipStream_t)stream, n,
                       (const uint16_t*)inp, (int8_t*)out);
    return launch_status();
}

int cpmk_copy_pos_hidden(int32_t batch, int32_t hidden_size, int32_t seq_len, int32_t pos, const void* inp, void* out, void* stream) {
    clear_stale_error();
    if (batch < 0 || hidden_size < 0 || seq_len < 0 || pos < 0 || (seq_len > 0 && pos >= seq_len)) return CPMK_EBADARG;
    if ((int64_t)batch * hidden_size * seq_len == 0) return 0;
    if (any_null(inp, out)) return CPMK_EBADARG;
    for (int64_t b0 = 0; b0 < batch; b0 += 65535) {       // (grid y: at most 65535 batch entries per launch)
        const int64_t nb = batch - b0 < 65535 ? batch - b0 : 65535;
        hipLaunchKernelGGL(k_copy_pos_hidden, dim3((unsigned)ceil_div(hidden_size, 256), (unsigned)nb), dim3(256), 0,
                           (hipStream_t)stream, hidden_size, seq_len, pos, (const half_t*)inp + b0 * hidden_size * seq_len,
                           (half_t*)out + b0 * hidden_size);
        if (int e = launch_status()) return e;
    }
    return 0;
}

}  // extern "C"
