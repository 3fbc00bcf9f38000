// Callers either side of the int8 path in a decode loop: token-embedding gathers and the copy
// of one step's hidden state into a key/value buffer.  Pure data movement (bit-exact).
//   embedding_forward : out[b, i, j] = weights[ids[b, j], i]        cuda/embedding.cu:6-37
//   embedding_step    : out[b, :]    = weights[ids[b], :]           cuda/embedding.cu:90-103
//   copy_data_to_kv   : out[b, pos, :] = in[b, :]                   cuda/utils.cu:13-29
#include "common.h"

namespace cpmk {

// 64 tokens x 64 hidden units per workgroup: rows of the table are read in 128-byte pieces,
// transposed through LDS and written as 128-byte pieces of the (hidden, seq) output.
__global__ __launch_bounds__(256) void k_embedding_forward(int32_t n, int32_t m, const int32_t* __restrict__ ids,
                                                           const half_t* __restrict__ weights,
                                                           half_t* __restrict__ out, int vec) {
    __shared__ half_t tile[64][64 + 2];      // [token][hidden]
    const int b = blockIdx.z;
    const int32_t j0 = blockIdx.x * 64, i0 = blockIdx.y * 64;
    const int tid = threadIdx.x;
    for (int q = tid; q < 64 * 8; q += 256) {
        const int jj = q >> 3, c = q & 7;
        const int32_t j = j0 + jj, i = i0 + c * 8;
        half8_t v;
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = (half_t)0.0f;
        if (j < m) {
            const half_t* row = weights + (int64_t)ids[(int64_t)b * m + j] * n;
            if (vec && i + 8 <= n) v = *reinterpret_cast<const half8_t*>(row + i);
            else
                for (int e = 0; e < 8; ++e)
                    if (i + e < n) v[e] = row[i + e];
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) tile[jj][c * 8 + e] = v[e];
    }
    __syncthreads();
    for (int q = tid; q < 64 * 64; q += 256) {
        const int ii = q >> 6, jj = q & 63;
        const int32_t i = i0 + ii, j = j0 + jj;
        if (i < n && j < m) out[((int64_t)b * n + i) * m + j] = tile[jj][ii];
    }
}

// One row per workgroup: 16-byte copies when the row allows it.
__global__ __launch_bounds__(256) void k_row_copy(int32_t n, const int32_t* __restrict__ ids, const half_t* __restrict__ src,
                                                  half_t* __restrict__ dst, int64_t dst_row_stride, int64_t dst_offset,
                                                  int vec) {
    const int64_t b = blockIdx.x;
    const half_t* s = src + (ids ? (int64_t)ids[b] : b) * n;
    half_t* d = dst + b * dst_row_stride + dst_offset;
    if (vec) {
        for (int32_t i = threadIdx.x; i < (n >> 3); i += 256)
            reinterpret_cast<half8_t*>(d)[i] = reinterpret_cast<const half8_t*>(s)[i];
    } else {
        for (int32_t i = threadIdx.x; i < n; i += 256) d[i] = s[i];
    }
}

}  // namespace cpmk

using namespace cpmk;

extern "C" {

int cpmk_embedding_forward(int32_t batch, int32_t hidden_size, int32_t seq_len, const void* ids, const void* weights,
                           void* out, void* stream) {
    clear_stale_error();
    if (batch < 0 || hidden_size < 0 || seq_len < 0) return CPMK_EBADARG;
    if ((int64_t)batch * hidden_size * seq_len == 0) return 0;
    if (any_null(ids, weights, out)) return CPMK_EBADARG;
    if (ceil_div(hidden_size, 64) > 65535) return CPMK_ETOOBIG;
    const int vec = (hidden_size % 8 == 0) && aligned16(weights);
    for (int64_t b0 = 0; b0 < batch; b0 += 65535) {       // (grid z: at most 65535 batch entries per launch)
        const int64_t nb = batch - b0 < 65535 ? batch - b0 : 65535;
        dim3 grid((unsigned)ceil_div(seq_len, 64), (unsigned)ceil_div(hidden_size, 64), (unsigned)nb);
        hipLaunchKernelGGL(k_embedding_forward, grid, dim3(256), 0, (hipStream_t)stream, hidden_size, seq_len,
                           (const int32_t*)ids + b0 * seq_len, (const half_t*)weights, (half_t*)out + b0 * hidden_size * seq_len, vec);
        if (int e = launch_status()) return e;
    }
    return 0;
}

int cpmk_embedding_step(int32_t batch, int32_t embedding_size, const void* ids, const void* weights, void* out,
                        void* stream) {
    clear_stale_error();
    if (batch < 0 || embedding_size < 0) return CPMK_EBADARG;
    if ((int64_t)batch * embedding_size == 0) return 0;
    if (any_null(ids, weights, out)) return CPMK_EBADARG;
    const int vec = (embedding_size % 8 == 0) && aligned16(weights) && aligned16(out);
    hipLaunchKernelGGL(k_row_copy, dim3((unsigned)batch), dim3(256), 0, (hipStream_t)stream, embedding_size,
                       (const int32_t*)ids, (const half_t*)weights, (half_t*)out, (int64_t)embedding_size, (int64_t)0, vec);
    return launch_status();
}

int cpmk_copy_data_to_kv(int32_t batch, int32_t buffer_len, int32_t n, const void* inp, void* out, int32_t pos,
                         void* stream) {
    clear_stale_error();
    if (batch < 0 || buffer_len < 0 || n < 0 || pos < 0 || pos >= buffer_len) return CPMK_EBADARG;
    if (n % 2) return CPMK_EALIGN;      // kernels/utils.py:25
    if ((int64_t)batch * n == 0) return 0;
    if (any_null(inp, out)) return CPMK_EBADARG;
    const int vec = (n % 8 == 0) && aligned16(inp) && aligned16(out);
    hipLaunchKernelGGL(k_row_copy, dim3((unsigned)batch), dim3(256), 0, (hipStream_t)stream, n, (const int32_t*)nullptr,
                       (const half_t*)inp, (half_t*)out, (int64_t)buffer_len * n, (int64_t)pos * n, vec);
    return launch_status();
}

}  // extern "C"
