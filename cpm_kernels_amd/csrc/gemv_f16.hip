// fp16 matrix-vector products of the decode loop (cuda/gemv.cu:78-175 and the cuBLASLt calls
// of kernels/gemv.py:82-283), fp32 accumulation, fp16 result:
//   gemv_fp16               out[b,o] = sum_k mat[b,o,k] * vec[b,k]
//   gemv_fp16_transpose     out[b,o] = sum_k mat[b,k,o] * vec[b,k]
//   gemv_broadcast_mat_fp16 out[b,o] = sum_k mat[o,k]   * vec[b,k]    (one matrix for all vectors)
// All three stream the matrix from HBM once.
#include "common.h"
#include <type_traits>

namespace cpmk {

constexpr int kShortLoads = 4;        // k_gemv_f16_short: loads in flight per lane when the grid still fills the chip
constexpr int kShortMinGroups = 2048; // ... which it does from eight workgroups a compute unit on
constexpr int kTransposeLoads = 8;    // k_gemv_f16_transpose: rows requested per lane before the first is used


// One wave per (batch, row): 16-byte loads of the row and of the vector, wave reduction.
// mat_bstride = 0 shares the matrix over the batch (then the rows of all vectors are done by one
// wave, so the matrix is still read once).
template <int NB>
__global__ __launch_bounds__(256) void k_gemv_f16_rows(int32_t batch, int32_t dim_out, int32_t dim_in, int64_t mat_bstride,
                                                       const half_t* __restrict__ mat, const half_t* __restrict__ vec,
                                                       half_t* __restrict__ out, int vec8) {
    const int lane = threadIdx.x & 63;
    const int64_t item = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    // private matrices: item = b*dim_out + row; shared matrix: item = row, all NB vectors of a pass
    const int64_t b0 = mat_bstride ? item / dim_out : (int64_t)blockIdx.y * NB;
    const int32_t row = (int32_t)(mat_bstride ? item - b0 * dim_out : item);
    if (row >= dim_out || b0 >= batch) return;
    const half_t* mrow = mat + b0 * mat_bstride + (int64_t)row * dim_in;
    float acc[NB];
#pragma unroll
    for (int t = 0; t < NB; ++t) acc[t] = 0.0f;
    if (vec8) {
        for (int32_t i = lane; i < (dim_in >> 3); i += 64) {
            const half8_t w = reinterpret_cast<const half8_t*>(mrow)[i];
#pragma unroll
            for (int t = 0; t < NB; ++t) {
                if (b0 + t < batch) {
                    const half8_t v = reinterpret_cast<const half8_t*>(vec + (b0 + t) * dim_in)[i];
#pragma unroll
                    for (int e = 0; e < 8; ++e) acc[t] = __builtin_fmaf((float)w[e], (float)v[e], acc[t]);
                }
            }
        }
    } else {
        for (int32_t i = lane; i < dim_in; i += 64) {
            const float w = (float)mrow[i];
#pragma unroll
            for (int t = 0; t < NB; ++t)
                if (b0 + t < batch) acc[t] = __builtin_fmaf(w, (float)vec[(b0 + t) * dim_in + i], acc[t]);
        }
    }
#pragma unroll
    for (int t = 0; t < NB; ++t) {
        const float s = wave_sum(acc[t]);
        if (lane == 0 && b0 + t < batch) out[(b0 + t) * dim_out + row] = (half_t)s;
    }
}

// Short rows (dim_in <= 256, the head dimension of attention scores over a key cache): LPRK lanes
// per row, one 16-byte piece each (LPRK >= dim_in / 8), so a wave covers 64 / LPRK consecutive rows
// with one coalesced load, and U such loads (U * 1 KB of consecutive rows) are in flight per wave
// before the first is used; the row sums are finished with LPRK-wide butterfly shuffles.  The matrix
// is read once and bypasses the caches' retention; the vectors are shared by dim_out rows and stay.
// item = b * dim_out + row.
template <int LPRK, int U>
__global__ __launch_bounds__(256) void k_gemv_f16_short(int64_t items, int32_t dim_out, int32_t dim_in,
                                                        const half_t* __restrict__ mat, const half_t* __restrict__ vec,
                                                        half_t* __restrict__ out) {
    constexpr int RPW = 64 / LPRK;
    const int lane = threadIdx.x & 63, pl = lane % LPRK;
    const int64_t item0 = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * (U * RPW) + lane / LPRK;
    const bool used = pl < (dim_in >> 3);
    half8_t w[U], x[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int64_t item = item0 + u * RPW;
        const int64_t it = item < items ? item : items - 1;
        const int64_t b = it / dim_out;
        if (used) {
            w[u] = __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(mat + it * dim_in) + pl);
            x[u] = reinterpret_cast<const half8_t*>(vec + b * dim_in)[pl];
        }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int64_t item = item0 + u * RPW;
        float acc = 0.0f;
        if (used) {
#pragma unroll
            for (int e = 0; e < 8; ++e) acc = __builtin_fmaf((float)w[u][e], (float)x[u][e], acc);
        }
#pragma unroll
        for (int o = 1; o < LPRK; o <<= 1) acc += __shfl_xor(acc, o, kWave);
        if (item < items && pl == 0) out[item] = (half_t)acc;
    }
}

// mat (batch, dim_in, dim_out): 256 threads = 32 row groups x 8 lanes of 8 adjacent columns; the
// row groups stride over dim_in and are combined in LDS.  A lane requests kTransposeLoads rows before it
// uses the first (the sums still run in row order); the matrix is read once and bypasses the caches'
// retention.  gridDim = (ceil(dim_out/64), batch).
__global__ __launch_bounds__(256) void k_gemv_f16_transpose(int32_t dim_out, int32_t dim_in, const half_t* __restrict__ mat,
                                                            const half_t* __restrict__ vec, half_t* __restrict__ out,
                                                            int vec8) {
    __shared__ float red[32][65];
    const int lane8 = threadIdx.x & 7, rg = threadIdx.x >> 3;
    const int32_t col0 = blockIdx.x * 64 + lane8 * 8;
    const int64_t b = blockIdx.y;
    const half_t* base = mat + b * dim_in * dim_out;
    const half_t* v = vec + b * dim_in;
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.0f;
    if (vec8) {
        if (col0 < dim_out) {
            const half_t* col = base + col0;
            int32_t i = rg;
            for (; i + 32 * (kTransposeLoads - 1) < dim_in; i += 32 * kTransposeLoads) {
                half8_t w[kTransposeLoads];
                float x[kTransposeLoads];
#pragma unroll
                for (int u = 0; u < kTransposeLoads; ++u) {
                    w[u] = __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(col + (int64_t)(i + 32 * u) * dim_out));
                    x[u] = (float)v[i + 32 * u];
                }
#pragma unroll
                for (int u = 0; u < kTransposeLoads; ++u)
#pragma unroll
                    for (int e = 0; e < 8; ++e) acc[e] = __builtin_fmaf(x[u], (float)w[u][e], acc[e]);
            }
            for (; i < dim_in; i += 32) {
                const half8_t w = __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(col + (int64_t)i * dim_out));
                const float x = (float)v[i];
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[e] = __builtin_fmaf(x, (float)w[e], acc[e]);
            }
        }
    } else {
        for (int32_t i = rg; i < dim_in; i += 32) {
            const float x = (float)v[i];
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (col0 + e < dim_out) acc[e] = __builtin_fmaf(x, (float)base[(int64_t)i * dim_out + col0 + e], acc[e]);
        }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) red[rg][lane8 * 8 + e] = acc[e];
    __syncthreads();
    if (threadIdx.x < 64) {
        float r = 0.0f;
#pragma unroll 8
        for (int g = 0; g < 32; ++g) r += red[g][threadIdx.x];
        const int32_t col = blockIdx.x * 64 + threadIdx.x;
        if (col < dim_out) out[b * dim_out + col] = (half_t)r;
    }
}

// One matrix for one or two vectors (decode with a batch of one or two sequences), rows of PPL * 512 halves: no
// matrix cores.  One workgroup of eight waves per compute unit; wave w takes rows w, w + 8, ... of the workgroup's
// share, R of them.  A row is PPL instructions of 1 KB in address order (16 bytes a lane); the loads of up to
// three rows (two of the long ones) are in flight per wave, the next row's requested before a row is used.
// Every lane keeps the vectors' halves at its positions in registers (in LDS, shared by the waves, when they
// are more than 16 pieces) and multiplies with v_dot2_f32_f16 (fp32
// sums, one chain per row and vector in a fixed order, so the result does not depend on timing); the lanes' sums
// are added over the wave, and the outputs leave through LDS so that a vector's outputs are stored contiguously.
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

__device__ inline float wave_sum_f32_to_lane63(float v) {
    auto from = [](float x, auto ctrl, auto rows, auto keep) {
        return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), decltype(ctrl)::value,
                                                                     decltype(rows)::value, 0xf, decltype(keep)::value));
    };
    using std::integral_constant;
    v += from(v, integral_constant<int, 0xB1>{}, integral_constant<int, 0xf>{}, integral_constant<bool, true>{});   // quad_perm [1,0,3,2]
    v += from(v, integral_constant<int, 0x4E>{}, integral_constant<int, 0xf>{}, integral_constant<bool, true>{});   // quad_perm [2,3,0,1]
    v += from(v, integral_constant<int, 0x141>{}, integral_constant<int, 0xf>{}, integral_constant<bool, true>{});  // row_half_mirror
    v += from(v, integral_constant<int, 0x140>{}, integral_constant<int, 0xf>{}, integral_constant<bool, true>{});  // row_mirror
    v += from(v, integral_constant<int, 0x142>{}, integral_constant<int, 0xa>{}, integral_constant<bool, false>{}); // row_bcast15 into rows 1 and 3
    v += from(v, integral_constant<int, 0x143>{}, integral_constant<int, 0xc>{}, integral_constant<bool, false>{}); // row_bcast31 into rows 2 and 3
    return v;                                                                                                       // the total: lane 63 only
}

template <int NV, int PPL, int R>
__global__ __launch_bounds__(512) void k_gemv_f16_rowwise(int32_t batch, int32_t dim_out, int32_t rpb, const half_t* __restrict__ mat,
                                                          const half_t* __restrict__ vec, half_t* __restrict__ out) {
    constexpr int DIN = PPL * 512;
    constexpr bool VLDS = NV * PPL > 16;           // the vectors' pieces in LDS instead of registers (rows of more than 4096 halves)
    constexpr int D = VLDS ? (R < 2 ? R : 2) : (R < 3 ? R : 3);      // rows in flight per wave
    __shared__ float part[8 * R * NV];             // [row of the share][vector]
    __shared__ __attribute__((aligned(16))) half8_t vlds[VLDS ? NV * PPL * 64 : 1];
    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int32_t row0 = blockIdx.x * rpb;
    // the vectors are requested first: they come from L2 and are there before the first row is
    half8_t vf[VLDS ? 1 : NV][VLDS ? 1 : PPL];
    constexpr int VPT = VLDS ? (NV * PPL * 64 + 511) / 512 : 1;     // pieces of the vectors a thread brings into LDS
    half8_t vstage[VPT];
    if constexpr (VLDS) {
#pragma unroll
        for (int j = 0; j < VPT; ++j) {
            const int piece = tid + j * 512;       // piece = (v * PPL + i) * 64 + lane of the reader
            const int v = piece / (PPL * 64), off = piece - v * (PPL * 64);
            if (piece < NV * PPL * 64) vstage[j] = *reinterpret_cast<const half8_t*>(vec + (uint32_t)min(v, batch - 1) * (uint32_t)DIN + off * 8);
        }
    } else {
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const half_t* vp = vec + (uint32_t)min(v, batch - 1) * (uint32_t)DIN + lane * 8;
#pragma unroll
            for (int i = 0; i < PPL; ++i) vf[v][i] = *reinterpret_cast<const half8_t*>(vp + i * 512);
        }
    }
    half8_t wf[D][PPL];
    auto request = [&](int r, half8_t (&buf)[PPL]) {
        const int32_t row = min(row0 + min(r * 8 + w, rpb - 1), dim_out - 1);       // (rows past the share repeat its last row)
        const half_t* rp = mat + (uint32_t)row * (uint32_t)DIN + lane * 8;
#pragma unroll
        for (int i = 0; i < PPL; ++i) buf[i] = __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(rp + i * 512));
    };
#pragma unroll
    for (int r = 0; r < D - 1; ++r) request(r, wf[r]);
    if constexpr (VLDS) {
#pragma unroll
        for (int j = 0; j < VPT; ++j)
            if (tid + j * 512 < NV * PPL * 64) vlds[tid + j * 512] = vstage[j];
        __syncthreads();
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (r + D - 1 < R) request(r + D - 1, wf[(r + D - 1) % D]);
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            float acc = 0.0f;
#pragma unroll
            for (int i = 0; i < PPL; ++i) {
                const half8_t a = wf[r % D][i];
                half8_t b;
                if constexpr (VLDS) b = vlds[(v * PPL + i) * 64 + lane];
                else b = vf[v][i];
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    acc = __builtin_amdgcn_fdot2(half2_t{a[2 * e], a[2 * e + 1]}, half2_t{b[2 * e], b[2 * e + 1]}, acc, false);
            }
            const float t = wave_sum_f32_to_lane63(acc);
            if (lane == 63) part[(r * 8 + w) * NV + v] = t;
        }
    }
    __syncthreads();
    const int obb = tid / rpb, orr = tid - obb * rpb;
    if (tid < rpb * NV) {
        const int32_t row = row0 + orr;
        if (row < dim_out && obb < batch) out[(int64_t)obb * dim_out + row] = (half_t)part[orr * NV + obb];
    }
}

// Takes the call when the shape fits the row-wise kernel: rows of 4096 or 10240 halves (the row lengths of the
// model this path serves), one or two vectors, 9 to 40 rows per compute unit ([10240, 4096], [4096, 4096] and
// [4096, 10240] among them).
static bool launch_gemv_f16_rowwise(int32_t batch, int32_t dim_out, int32_t dim_in, const half_t* mat, const half_t* vec,
                                    half_t* out, hipStream_t st) {
    if (batch > 2 || (dim_in != 4096 && dim_in != 10240) || (int64_t)dim_out * dim_in * 2 >= (1ll << 32) || !aligned16(mat) || !aligned16(vec))
        return false;
    const int64_t rpb = ceil_div(dim_out, compute_units());
    const int r = (int)ceil_div(rpb, 8);
    if (r < 2 || r > 5) return false;
    const dim3 grid((unsigned)ceil_div(dim_out, rpb));
    auto go = [&](auto kern) { hipLaunchKernelGGL(kern, grid, dim3(512), 0, st, batch, dim_out, (int32_t)rpb, mat, vec, out); };
    auto pick = [&](auto nvc, auto pplc) {
        constexpr int NV = decltype(nvc)::value, PPL = decltype(pplc)::value;
        if (r == 2) go(k_gemv_f16_rowwise<NV, PPL, 2>);
        else if (r == 3) go(k_gemv_f16_rowwise<NV, PPL, 3>);
        else if (r == 4) go(k_gemv_f16_rowwise<NV, PPL, 4>);
        else go(k_gemv_f16_rowwise<NV, PPL, 5>);
    };
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    if (dim_in == 4096) {
        if (batch == 1) pick(I1{}, std::integral_constant<int, 8>{});
        else pick(I2{}, std::integral_constant<int, 8>{});
    } else {
        if (batch == 1) pick(I1{}, std::integral_constant<int, 20>{});
        else pick(I2{}, std::integral_constant<int, 20>{});
    }
    return true;
}

}  // namespace cpmk

using namespace cpmk;

extern "C" {

int cpmk_gemv_fp16(int32_t batch, int32_t dim_out, int32_t dim_in, const void* mat, const void* vec, void* out,
                   void* stream) {
    clear_stale_error();
    if (batch < 0 || dim_out < 0 || dim_in < 0) return CPMK_EBADARG;
    if ((int64_t)batch * dim_out == 0) return 0;
    if (out == nullptr || (dim_in > 0 && any_null(mat, vec))) return CPMK_EBADARG;
    const int vec8 = (dim_in % 8 == 0) && aligned16(mat) && aligned16(vec);
    const int64_t items = (int64_t)batch * dim_out;
    if (!grid_fits(ceil_div(items, 4))) return CPMK_ETOOBIG;
    if (vec8 && dim_in <= 256) {
        const int p = dim_in >> 3;                      // 16-byte pieces per row
        const hipStream_t st = (hipStream_t)stream;
        auto go = [&](auto lc) {
            constexpr int L = decltype(lc)::value;
            constexpr int per_wave = 64 / L;             // rows of one load
            if (items >= (int64_t)kShortMinGroups * 4 * kShortLoads * per_wave)     // enough rows for several workgroups a compute unit
                hipLaunchKernelGGL((k_gemv_f16_short<L, kShortLoads>), dim3((unsigned)ceil_div(items, 4 * kShortLoads * per_wave)), dim3(256), 0, st, items,
                                   dim_out, dim_in, (const half_t*)mat, (const half_t*)vec, (half_t*)out);
            else
                hipLaunchKernelGGL((k_gemv_f16_short<L, 1>), dim3((unsigned)ceil_div(items, 4 * per_wave)), dim3(256), 0, st, items, dim_out,
                                   dim_in, (const half_t*)mat, (const half_t*)vec, (half_t*)out);
        };
        if (p <= 1) go(std::integral_constant<int, 1>{});
        else if (p <= 2) go(std::integral_constant<int, 2>{});
        else if (p <= 4) go(std::integral_constant<int, 4>{});
        else if (p <= 8) go(std::integral_constant<int, 8>{});
        else if (p <= 16) go(std::integral_constant<int, 16>{});
        else go(std::integral_constant<int, 32>{});
        return launch_status();
    }
    hipLaunchKernelGGL((k_gemv_f16_rows<1>), dim3((unsigned)ceil_div(items, 4)), dim3(256), 0, (hipStream_t)stream, batch,
                       dim_out, dim_in, (int64_t)dim_out * dim_in, (const half_t*)mat, (const half_t*)vec, (half_t*)out, vec8);
    return launch_status();
}

int cpmk_gemv_fp16_transpose(int32_t batch, int32_t dim_out, int32_t dim_in, const void* mat, const void* vec, void* out,
                             void* stream) {
    clear_stale_error();
    if (batch < 0 || dim_out < 0 || dim_in < 0) return CPMK_EBADARG;
    if ((int64_t)batch * dim_out == 0) return 0;
    if (out == nullptr || (dim_in > 0 && any_null(mat, vec))) return CPMK_EBADARG;
    const int vec8 = (dim_out % 8 == 0) && aligned16(mat);
    for (int64_t b0 = 0; b0 < batch; b0 += 65535) {       // (grid y: at most 65535 batch entries per launch)
        const int64_t nb = batch - b0 < 65535 ? batch - b0 : 65535;
        dim3 grid((unsigned)ceil_div(dim_out, 64), (unsigned)nb);
        hipLaunchKernelGGL(k_gemv_f16_transpose, grid, dim3(256), 0, (hipStream_t)stream, dim_out, dim_in,
                           (const half_t*)mat + b0 * dim_in * dim_out, (const half_t*)vec + b0 * dim_in, (half_t*)out + b0 * dim_out, vec8);
        if (int e = launch_status()) return e;
    }
    return 0;
}

int cpmk_gemv_broadcast_mat_fp16(int32_t batch, int32_t dim_out, int32_t dim_in, const void* mat, const void* vec,
                                 void* out, void* stream) {
    clear_stale_error();
    if (batch < 0 || dim_out < 0 || dim_in < 0) return CPMK_EBADARG;
    if ((int64_t)batch * dim_out == 0) return 0;
    if (out == nullptr || (dim_in > 0 && any_null(mat, vec))) return CPMK_EBADARG;
    if (launch_gemv_f16_rowwise(batch, dim_out, dim_in, (const half_t*)mat, (const half_t*)vec, (half_t*)out, (hipStream_t)stream))
        return launch_status();
    {   // matrix cores when the rows are whole 256-byte chunks
        const int rc = gemv_f16_coalesced(batch, dim_out, dim_in, mat, vec, out, (hipStream_t)stream);
        if (rc >= 0) return rc;
    }
    if (dim_in >= 128) {   // other row lengths: the predicated matrix-core kernel (short rows stay on the wave-per-row kernel below)
        const int rc = gemv_f16_mfma(batch, dim_out, dim_in, mat, vec, out, (hipStream_t)stream);
        if (rc >= 0) return rc;
    }
    const int vec8 = (dim_in % 8 == 0) && aligned16(mat) && aligned16(vec);
    constexpr int NB = 8;               // vectors per pass over a matrix row
    const int64_t passes = ceil_div(batch, NB);
    if (passes > 65535) return CPMK_ETOOBIG;
    dim3 grid((unsigned)ceil_div(dim_out, 4), (unsigned)passes);
    hipLaunchKernelGGL((k_gemv_f16_rows<NB>), grid, dim3(256), 0, (hipStream_t)stream, batch, dim_out, dim_in, (int64_t)0,
                       (const half_t*)mat, (const half_t*)vec, (half_t*)out, vec8);
    return launch_status();
}

}  // extern "C"
