// T5-style relative position buckets and the bias gather built on them
// (cuda/position_bucket.cu:6-54, :105-133 of the reference).
#include "common.h"

namespace cpmk {

// int32 table of max_distance entries.  Same float formulation as cu_init_position_mapping:
// note that max_distance / exact_buckets is an integer division there (.cu:16).
__global__ __launch_bounds__(256) void k_position_init(int32_t num_buckets, int32_t max_distance, int32_t* out,
                                                       int bidirectional) {
    const int32_t part = num_buckets / (bidirectional ? 2 : 1);
    const int32_t exact = part / 2;
    const int32_t log_buckets = part - exact;
    const float v = logf((float)(max_distance / exact));
    for (int32_t i = blockIdx.x * 256 + threadIdx.x; i < max_distance; i += gridDim.x * 256) {
        if (i < exact) out[i] = i;
        else out[i] = (int32_t)(logf((float)i / (float)exact) / v * (float)log_buckets) + exact;
    }
}

__device__ inline int32_t bucket_of(int32_t rel, int32_t num_buckets, int32_t max_distance,
                                    const int32_t* __restrict__ table, int bidirectional) {
    int32_t off = 0;
    if (rel < 0) {
        if (bidirectional) { rel = -rel; off = num_buckets / 2; }
        else rel = 0;
    }
    if (rel >= max_distance) rel = max_distance - 1;
    return table[rel] + off;
}

// out[h, k, q] = weight[h, bucket(q - k)].  The bias is Toeplitz: for one head it depends on
// q - k only.  A workgroup builds that head's diagonal vector d[r], r = q - k + (key_len-1),
// for the q - k range of its KR key rows in LDS and then streams the rows out.
// Long rows are cut into pieces of at most QC queries, each with a diagonal of its own.
// grid = (ceil(key_len / KR), num_heads, ceil(query_len / QC))
constexpr int KR = 16;
constexpr int QC = 16384;
__global__ __launch_bounds__(256) void k_position_forward(int32_t query_len, int32_t key_len, int32_t num_buckets,
                                                          int32_t max_distance, const int32_t* __restrict__ table,
                                                          const half_t* __restrict__ weight, half_t* out,
                                                          int bidirectional, int vec8) {
    extern __shared__ half_t diag[];          // min(query_len, QC) + KR - 1 entries
    const int32_t k0 = blockIdx.x * KR;
    const int32_t h = blockIdx.y;
    const int32_t q0 = blockIdx.z * QC;
    const int32_t nq = min(QC, query_len - q0);
    const int32_t kend = min(k0 + KR, key_len);
    // diag[t] holds the weight of rel = rel_min + t; rel = q - k ranges over [q0 - (kend-1), q0 + nq - 1 - k0]
    const int32_t rel_min = q0 - (kend - 1);
    const int32_t nd = nq + (kend - k0) - 1;
    const half_t* wh = weight + (int64_t)h * num_buckets;
    for (int32_t t = threadIdx.x; t < nd; t += 256)
        diag[t] = wh[bucket_of(rel_min + t, num_buckets, max_distance, table, bidirectional)];
    __syncthreads();
    if (vec8) {
        // 16-byte stores: the workgroup's rows are cut into pieces of eight queries and dealt to the threads
        const int32_t nv = nq >> 3, items = (kend - k0) * nv;
        for (int32_t it = threadIdx.x; it < items; it += 256) {
            const int32_t kk = it / nv, qv = it - kk * nv;
            const int32_t k = k0 + kk;
            const half_t* d = diag + (qv * 8 + q0 - k - rel_min);
            half8_t v;
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = d[e];
            *reinterpret_cast<half8_t*>(out + ((int64_t)h * key_len + k) * query_len + q0 + qv * 8) = v;
        }
        return;
    }
    for (int32_t k = k0; k < kend; ++k) {
        half_t* orow = out + ((int64_t)h * key_len + k) * query_len + q0;
        const int32_t shift = q0 - k - rel_min;    // q - k - rel_min = (q - q0) + shift
        for (int32_t q = threadIdx.x; q < nq; q += 256) orow[q] = diag[q + shift];
    }
}

// out[h, k] for one query position (decode step).
__global__ __launch_bounds__(256) void k_position_step(int32_t query_pos, int32_t key_len, int32_t num_buckets,
                                                       int32_t max_distance, int32_t num_heads,
                                                       const int32_t* __restrict__ table,
                                                       const half_t* __restrict__ weight, half_t* out,
                                                       int bidirectional) {
    const int32_t k = blockIdx.x * 256 + threadIdx.x;
    if (k >= key_len) return;
    const int32_t bucket = bucket_of(query_pos - k, num_buckets, max_distance, table, bidirectional);
    for (int32_t h = 0; h < num_heads; ++h) out[(int64_t)h * key_len + k] = weight[(int64_t)h * num_buckets + bucket];
}

}  // namespace cpmk

using namespace cpmk;

extern "C" {

int cpmk_position_embedding_init(int32_t num_buckets, int32_t max_distance, void* out, int bidirectional,
                                 void* stream) {
    clear_stale_error();
    if (num_buckets < (bidirectional ? 4 : 2) || max_distance < 0) return CPMK_EBADARG;
    if (max_distance == 0) return 0;
    if (out == nullptr) return CPMK_EBADARG;
    hipLaunchKernelGGL(k_position_init, dim3((unsigned)ceil_div(max_distance, 256)), dim3(256), 0,
                       (hipStream_t)stream, num_buckets, max_distance, (int32_t*)out, bidirectional);
    return launch_status();
}

int cpmk_position_embedding_forward(int32_t query_len, int32_t key_len, int32_t num_buckets, int32_t max_distance,
                                    int32_t num_heads, const void* position_mapping, const void* weight, void* out,
                                    int bidirectional, void* stream) {
    clear_stale_error();
    if (query_len < 0 || key_len < 0 || num_heads < 0 || num_buckets <= 0 || max_distance <= 0) return CPMK_EBADARG;
    if ((int64_t)query_len * key_len * num_heads == 0) return 0;
    if (any_null(position_mapping, weight, out)) return CPMK_EBADARG;
    const size_t smem = (size_t)((query_len < QC ? query_len : QC) + KR - 1) * sizeof(half_t);
    const int vec8 = (query_len % 8 == 0) && aligned16(out);       // every row then starts on a 16-byte boundary
    // heads are the grid's y dimension (at most 65535): more go out in several launches
    for (int64_t h0 = 0; h0 < num_heads; h0 += 65535) {
        const int64_t nh = num_heads - h0 < 65535 ? num_heads - h0 : 65535;
        dim3 grid((unsigned)ceil_div(key_len, KR), (unsigned)nh, (unsigned)ceil_div(query_len, QC));
        hipLaunchKernelGGL(k_position_forward, grid, dim3(256), smem, (hipStream_t)stream, query_len, key_len,
                           num_buckets, max_distance, (const int32_t*)position_mapping,
                           (const half_t*)weight + h0 * num_buckets, (half_t*)out + h0 * key_len * query_len, bidirectional, vec8);
        if (int e = launch_status()) return e;
    }
    return 0;
}

int cpmk_position_embedding_step(int32_t query_pos, int32_t key_len, int32_t num_buckets, int32_t max_distance,
                                 int32_t num_heads, const void* position_mapping, const void* weight, void* out,
                                 int bidirectional, void* stream) {
    clear_stale_error();
    if (key_len < 0 || num_heads < 0 || num_buckets <= 0 || max_distance <= 0) return CPMK_EBADARG;
    if ((int64_t)key_len * num_heads == 0) return 0;
    if (any_null(position_mapping, weight, out)) return CPMK_EBADARG;
    hipLaunchKernelGGL(k_position_step, dim3((unsigned)ceil_div(key_len, 256)), dim3(256), 0, (hipStream_t)stream,
                       query_pos, key_len, num_buckets, max_distance, num_heads, (const int32_t*)position_mapping,
                       (const half_t*)weight, (half_t*)out, bidirectional);
    return launch_status();
}

}  // extern "C"
