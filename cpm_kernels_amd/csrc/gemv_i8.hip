// Decode GEMV with a broadcast int8 weight matrix:
//   out[b,o] = fp16( (f32(sum_k mat[o,k]*vec[b,k]) * f32(scale_vec[b])) * f32(scale_mat[o]) )
// (cuda/gemv.cu:57-76 of the reference, which launches one 1024-thread block per output
// scalar and re-reads the weight row once per batch element).
//
// Here the weight matrix is streamed from HBM exactly once: the batch of quantised vectors
// is the second operand of v_mfma_i32_16x16x64_i8, so one pass over a 16-row slab of the
// matrix serves up to 128 vectors.  The sum over k is an exact integer sum, so splitting k
// over waves and reordering it inside the MFMA cannot change the int32 result.
//
// Loading the matrix directly in the MFMA register layout (lane = row) would make every lane of
// a load instruction touch a different cache line: 64 L1 lookups per instruction, and the vector
// L1 becomes the bottleneck at about a quarter of the HBM rate.  The fast kernel therefore loads
// 4 rows x 256 contiguous bytes per instruction (8 cache lines) and transposes 16-row groups
// into the MFMA layout through 4 KB of wave-private, XOR-swizzled LDS.
#include "common.h"
#include <atomic>
#include <type_traits>


namespace cpmk {

// Predicated MFMA kernel for dim_in % 16 == 0 that is not a multiple of 256 (loads in the MFMA
// layout, zero-filled past the end of k).
// Workgroup = NW waves, RG*16 consecutive matrix rows, all of k.  k is cut into 256-byte
// chunks dealt round-robin to the waves; a chunk is four 64-byte pieces, one MFMA each, and
// in piece j lane (r = l%16, q = l/16) reads bytes [j*64 + q*16, +16) of row r -- the four
// lanes of a row read one contiguous 64-byte sector per instruction.  The vector operand uses
// the same lane -> k assignment, which is all the MFMA needs.
// DW: rows that are only 4-byte aligned (dim_in % 16 != 0): a lane's 16 bytes still come in one load where they lie
// inside the row, as single dwords (zero past the end of k) across its end.
// F16: the same on fp16 data (cpmk_gemv_broadcast_mat_fp16 with rows that are not whole 256-byte chunks): dim_in is the
// row length in BYTES, a lane's 16 bytes are 8 halves of K for v_mfma_f32_16x16x32_f16, the accumulators are fp32 and
// leave without scales; the waves' partial sums are added in wave order.
template <int NW, int RG, int NB, bool DW = false, bool F16 = false>
__global__ __launch_bounds__(NW * 64) void k_gemv_mfma(int32_t batch, int32_t dim_out, int32_t dim_in,
                                                       const half_t* __restrict__ scale_mat,
                                                       const int8_t* __restrict__ mat,
                                                       const half_t* __restrict__ scale_vec,
                                                       const int8_t* __restrict__ vec,
                                                       half_t* __restrict__ out) {
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int r = lane & 15, q = lane >> 4;
    const int32_t row0 = blockIdx.x * (RG * 16);

    using acc_t = std::conditional_t<F16, float4_t, int4_t>;
    acc_t acc[RG][NB];
#pragma unroll
    for (int g = 0; g < RG; ++g)
#pragma unroll
        for (int t = 0; t < NB; ++t)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[g][t][e] = 0;

    const int nchunks = (dim_in + 255) >> 8;
    auto piece = [&](const int8_t* rowp, int32_t k0) __attribute__((always_inline)) {      // bytes [k0, k0 + 16) of a row, zeros past dim_in
        int4_t v = {0, 0, 0, 0};
        if constexpr (DW) {
            if (k0 + 16 <= dim_in) {       // (a global load of four dwords needs dword alignment only)
                struct __attribute__((aligned(4))) Int4Dword { int32_t x, y, z, w; };
                const Int4Dword t = *reinterpret_cast<const Int4Dword*>(rowp + k0);
                v = int4_t{t.x, t.y, t.z, t.w};
            } else {
#pragma unroll
                for (int d = 0; d < 3; ++d)
                    if (k0 + 4 * d < dim_in) v[d] = *reinterpret_cast<const int32_t*>(rowp + k0 + 4 * d);
            }
        } else {
            if (k0 < dim_in) v = *reinterpret_cast<const int4_t*>(rowp + k0);
        }
        return v;
    };
    for (int c = w; c < nchunks; c += NW) {
        const int32_t kb = c * 256 + q * 16;
        int4_t wv[RG][4], vv[NB][4];
#pragma unroll
        for (int g = 0; g < RG; ++g) {
            const int32_t row = row0 + g * 16 + r;
            const int8_t* p = mat + (int64_t)min(row, dim_out - 1) * dim_in;
#pragma unroll
            for (int j = 0; j < 4; ++j) wv[g][j] = row < dim_out ? piece(p, kb + j * 64) : int4_t{0, 0, 0, 0};
        }
#pragma unroll
        for (int t = 0; t < NB; ++t) {
            const int32_t b = t * 16 + r;
            const int8_t* p = vec + (int64_t)min(b, batch - 1) * dim_in;
#pragma unroll
            for (int j = 0; j < 4; ++j) vv[t][j] = b < batch ? piece(p, kb + j * 64) : int4_t{0, 0, 0, 0};
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int g = 0; g < RG; ++g)
#pragma unroll
                for (int t = 0; t < NB; ++t) {
                    if constexpr (F16)
                        acc[g][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, wv[g][j]), __builtin_bit_cast(half8_t, vv[t][j]),
                                                                           acc[g][t], 0, 0, 0);
                    else
                        acc[g][t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wv[g][j], vv[t][j], acc[g][t], 0, 0, 0);
                }
    }

    if constexpr (F16) {
        // every wave leaves its partial sums in a slice of its own; the output threads add the NW slices in wave order
        __shared__ float fslice[NW * RG * NB * 256];
#pragma unroll
        for (int g = 0; g < RG; ++g)
#pragma unroll
            for (int t = 0; t < NB; ++t)
#pragma unroll
                for (int e = 0; e < 4; ++e) fslice[(w * RG * NB + g * NB + t) * 256 + (q * 4 + e) * 16 + r] = acc[g][t][e];
        __syncthreads();
        for (int idx = tid; idx < RG * NB * 256; idx += NW * 64) {
            const int rr = idx % (RG * 16), bb = idx / (RG * 16);
            const int g = rr >> 4, t = bb >> 4;
            float sum = 0.0f;
#pragma unroll
            for (int ww = 0; ww < NW; ++ww) sum += fslice[(ww * RG * NB + g * NB + t) * 256 + (rr & 15) * 16 + (bb & 15)];
            const int32_t row = row0 + rr;
            if (row < dim_out && bb < batch) out[(int64_t)bb * dim_out + row] = (half_t)sum;
        }
        return;
    }
    __shared__ int32_t part[RG * NB][256];   // cross-wave sums (LDS integer atomics)
    for (int idx = tid; idx < RG * NB * 256; idx += NW * 64) (&part[0][0])[idx] = 0;
    __syncthreads();
    // accumulator e of lane l: matrix row (l/16)*4 + e, vector l%16 of the 16x16 tile
#pragma unroll
    for (int g = 0; g < RG; ++g)
#pragma unroll
        for (int t = 0; t < NB; ++t)
#pragma unroll
            for (int e = 0; e < 4; ++e) atomicAdd(&part[g * NB + t][(q * 4 + e) * 16 + r], (int32_t)acc[g][t][e]);
    __syncthreads();

    // part[tile][row_in_tile*16 + b_in_tile]; thread -> (b, row) with row fastest so a
    // vector's outputs are stored contiguously.
    for (int idx = tid; idx < RG * NB * 256; idx += NW * 64) {
        const int rr = idx % (RG * 16), bb = idx / (RG * 16);
        const int g = rr >> 4, t = bb >> 4;
        const int32_t s = part[g * NB + t][(rr & 15) * 16 + (bb & 15)];
        const int32_t row = row0 + rr;
        if (row < dim_out && bb < batch)
            out[(int64_t)bb * dim_out + row] = dequant(s, (float)scale_vec[bb], (float)scale_mat[row]);
    }
}

// Fast kernel: dim_in % 256 == 0.  Workgroup = NW waves and 4*r4 consecutive matrix rows (r4 <=
// 4*RG; the launcher sizes r4 so that every compute unit gets one workgroup); the 256-byte K
// chunks are dealt round-robin to the waves, two per trip so that a wave has both chunks' loads
// in flight before it touches either.  Per chunk a wave loads, fully coalesced, its rows and
// NB*16 vectors (lane l: 16-byte chunk l%16 of row l/16 + 4i), then turns each 16-row group into
// four MFMA operands (piece j: lane (r = l%16, q = l/16) holds bytes [j*64 + q*16, +16) of row r)
// by writing it to LDS at row*256 + ((chunk ^ row) << 4) and reading it back transposed; both
// directions are bank-conflict free.  LDS executes one wave's operations in order, so the 4 KB
// buffer is reused without waits.  Vectors past the end are clamped and row steps past r4 are
// not loaded (the MFMA then sees stale LDS bytes): both only feed outputs that are never stored.
//
// F16: the same kernel on fp16 data (cpmk_gemv_broadcast_mat_fp16): dim_in is then the row length in
// BYTES, a lane's 16 bytes are 8 halves of K for v_mfma_f32_16x16x32_f16 (the same lane -> byte
// assignment as the int8 instruction), the accumulators are fp32 and leave without scales.
// The matrix is read once and bypasses the caches' retention (the vectors, which every workgroup reads, stay).
template <int NW, int RG, int NB, bool F16 = false>
__global__ __launch_bounds__(NW * 64) void k_gemv_coalesced(int32_t batch, int32_t dim_out, int32_t dim_in, int32_t r4,
                                                            const half_t* __restrict__ scale_mat,
                                                            const int8_t* __restrict__ mat,
                                                            const half_t* __restrict__ scale_vec,
                                                            const int8_t* __restrict__ vec,
                                                            half_t* __restrict__ out) {
    __shared__ __attribute__((aligned(16))) int8_t tbuf[NW][4096];
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int r = lane & 15, q = lane >> 4;      // MFMA layout
    const int x = lane & 15, y4 = lane >> 4;     // load layout
    const int32_t rpb = r4 * 4;                  // rows of this workgroup
    const int32_t row0 = blockIdx.x * rpb;
    int8_t* tb = tbuf[w];
    // the scales of the outputs this thread will write, requested first so that they arrive with
    // the weights instead of costing a round trip to memory after the reduction
    constexpr int NOUT = (RG * NB * 256 + NW * 64 - 1) / (NW * 64);
    half_t osv[NOUT], osm[NOUT];
#pragma unroll
    for (int o = 0; o < NOUT; ++o) {
        const int idx = tid + o * NW * 64;
        const int rr = idx % rpb, bb = idx / rpb;
        osv[o] = osm[o] = (half_t)1.0f;
        if (!F16) {
            osv[o] = scale_vec[min(bb, batch - 1)];
            osm[o] = scale_mat[min(row0 + rr, dim_out - 1)];
        }
    }
    int woff[4], roff[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int yy = i * 4 + y4;
        woff[i] = yy * 256 + ((x ^ yy) << 4);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) roff[j] = r * 256 + (((j * 4 + q) ^ r) << 4);
    // 32-bit byte offsets from the two base pointers (the launcher checks that they fit)
    uint32_t wo[RG][4], vo[NB][4];
    bool wok[RG][4];
#pragma unroll
    for (int g = 0; g < RG; ++g)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int32_t row = row0 + (g * 4 + i) * 4 + y4;
            wok[g][i] = (g * 4 + i) < r4;
            wo[g][i] = (uint32_t)min(row, dim_out - 1) * (uint32_t)dim_in + x * 16;
        }
#pragma unroll
    for (int t = 0; t < NB; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) vo[t][i] = (uint32_t)min(t * 16 + i * 4 + y4, batch - 1) * (uint32_t)dim_in + x * 16;

    using acc_t = std::conditional_t<F16, float4_t, int4_t>;
    acc_t acc[RG][NB];
#pragma unroll
    for (int g = 0; g < RG; ++g)
#pragma unroll
        for (int t = 0; t < NB; ++t)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[g][t][e] = 0;

    auto load_chunk = [&](int4_t (&wr)[RG][4], int4_t (&vr)[NB][4], int c) __attribute__((always_inline)) {
#pragma unroll
        for (int g = 0; g < RG; ++g)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                wr[g][i] = int4_t{0, 0, 0, 0};
                if (wok[g][i]) wr[g][i] = __builtin_nontemporal_load(reinterpret_cast<const int4_t*>(mat + (wo[g][i] + (uint32_t)c * 256u)));
            }
#pragma unroll
        for (int t = 0; t < NB; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) vr[t][i] = *reinterpret_cast<const int4_t*>(vec + (vo[t][i] + (uint32_t)c * 256u));
    };
    auto mac_chunk = [&](int4_t (&wr)[RG][4], int4_t (&vr)[NB][4]) __attribute__((always_inline)) {
#pragma unroll
        for (int g = 0; g < RG; ++g) {
#pragma unroll
            for (int i = 0; i < 4; ++i) *reinterpret_cast<int4_t*>(tb + woff[i]) = wr[g][i];
#pragma unroll
            for (int j = 0; j < 4; ++j) wr[g][j] = *reinterpret_cast<const int4_t*>(tb + roff[j]);
        }
#pragma unroll
        for (int t = 0; t < NB; ++t) {
#pragma unroll
            for (int i = 0; i < 4; ++i) *reinterpret_cast<int4_t*>(tb + woff[i]) = vr[t][i];
#pragma unroll
            for (int j = 0; j < 4; ++j) vr[t][j] = *reinterpret_cast<const int4_t*>(tb + roff[j]);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int g = 0; g < RG; ++g)
#pragma unroll
                for (int t = 0; t < NB; ++t) {
                    if constexpr (F16)
                        acc[g][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, wr[g][j]),
                                                                           __builtin_bit_cast(half8_t, vr[t][j]), acc[g][t], 0, 0, 0);
                    else
                        acc[g][t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wr[g][j], vr[t][j], acc[g][t], 0, 0, 0);
                }
    };

    const int nchunks = dim_in >> 8;
    int c = w;
    if constexpr (RG + NB <= 5) {      // two chunks in flight where the registers allow it
        for (; c + NW < nchunks; c += 2 * NW) {
            int4_t wa[RG][4], va[NB][4], wb[RG][4], vb[NB][4];
            load_chunk(wa, va, c);
            load_chunk(wb, vb, c + NW);
            mac_chunk(wa, va);
            mac_chunk(wb, vb);
        }
    }
    for (; c < nchunks; c += NW) {
        int4_t wa[RG][4], va[NB][4];
        load_chunk(wa, va, c);
        mac_chunk(wa, va);
    }

    // thread -> (vector, row) with the row fastest, so a vector's outputs are stored contiguously
    if constexpr (F16) {
        // every wave leaves its partial sums in a slice of its own; the output threads add the NW slices in
        // wave order, so the result does not depend on timing
        __shared__ float fslice[NW * RG * NB * 256];
#pragma unroll
        for (int g = 0; g < RG; ++g)
#pragma unroll
            for (int t = 0; t < NB; ++t)
#pragma unroll
                for (int e = 0; e < 4; ++e) fslice[(w * RG * NB + g * NB + t) * 256 + (q * 4 + e) * 16 + r] = acc[g][t][e];
        __syncthreads();
#pragma unroll
        for (int o = 0; o < NOUT; ++o) {
            const int idx = tid + o * NW * 64;
            if (idx < rpb * NB * 16) {
                const int rr = idx % rpb, bb = idx / rpb;
                const int g = rr >> 4, t = bb >> 4;
                float s = 0.0f;
#pragma unroll
                for (int ww = 0; ww < NW; ++ww) s += fslice[(ww * RG * NB + g * NB + t) * 256 + (rr & 15) * 16 + (bb & 15)];
                const int32_t row = row0 + rr;
                if (row < dim_out && bb < batch) out[(int64_t)bb * dim_out + row] = (half_t)s;
            }
        }
    } else {
        __shared__ int32_t part[RG * NB][256];
        for (int idx = tid; idx < RG * NB * 256; idx += NW * 64) (&part[0][0])[idx] = 0;
        __syncthreads();
        // accumulator e of lane l: matrix row (l/16)*4 + e, vector l%16 of the 16x16 tile
#pragma unroll
        for (int g = 0; g < RG; ++g)
#pragma unroll
            for (int t = 0; t < NB; ++t)
#pragma unroll
                for (int e = 0; e < 4; ++e) atomicAdd(&part[g * NB + t][(q * 4 + e) * 16 + r], (int32_t)acc[g][t][e]);
        __syncthreads();
#pragma unroll
        for (int o = 0; o < NOUT; ++o) {
            const int idx = tid + o * NW * 64;
            if (idx < rpb * NB * 16) {
                const int rr = idx % rpb, bb = idx / rpb;
                const int g = rr >> 4, t = bb >> 4;
                const int32_t s = part[g * NB + t][(rr & 15) * 16 + (bb & 15)];
                const int32_t row = row0 + rr;
                if (row < dim_out && bb < batch) out[(int64_t)bb * dim_out + row] = dequant(s, (float)osv[o], (float)osm[o]);
            }
        }
    }
}

// One or two vectors (decode with a batch of one or two sequences): no matrix cores.  A wave reads whole rows --
// instruction i of a row brings bytes [1024 i, 1024 i + 1024), 16 per lane, whole cache lines in address order,
// the access pattern in which a one-round read of this size is quickest -- and multiplies them with v_dot4_i32_i8 against the vectors' bytes at the same positions,
// which every lane keeps in registers (NV x PPL pieces of 16 bytes).  One workgroup per compute unit, wave w
// takes rows w, w + 8, ... of the workgroup's share (G of them), all loads of a wave requested at once (G rows of
// PPL pieces, at most 20 pieces = 80 registers); the per-lane sums of a (row, vector) pair are added over the wave,
// and the outputs leave through LDS so that a vector's outputs are stored contiguously.
template <int NV, int PPL, int G>
__global__ __launch_bounds__(512) void k_gemv_rowwise(int32_t batch, int32_t dim_out, int32_t rpb,
                                                      const half_t* __restrict__ scale_mat,
                                                      const int8_t* __restrict__ mat,
                                                      const half_t* __restrict__ scale_vec,
                                                      const int8_t* __restrict__ vec,
                                                      half_t* __restrict__ out) {
    static_assert(G * PPL <= 20 && NV * PPL <= 20, "registers");
    constexpr int DIN = PPL * 1024;
    __shared__ int32_t part[8 * G * NV];           // [row of the share][vector]
    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int32_t row0 = blockIdx.x * rpb;
    int4_t wf[G][PPL];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const int32_t row = min(row0 + min(g * 8 + w, rpb - 1), dim_out - 1);       // (rows past the share repeat its last row)
        const int8_t* rp = mat + (uint32_t)row * (uint32_t)DIN + lane * 16;
#pragma unroll
        for (int i = 0; i < PPL; ++i) wf[g][i] = __builtin_nontemporal_load(reinterpret_cast<const int4_t*>(rp + i * 1024));
    }
    int4_t vf[NV][PPL];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int8_t* vp = vec + (uint32_t)min(v, batch - 1) * (uint32_t)DIN + lane * 16;
#pragma unroll
        for (int i = 0; i < PPL; ++i) vf[v][i] = *reinterpret_cast<const int4_t*>(vp + i * 1024);
    }
    // the outputs this thread will write and their scales (row fastest: a vector's outputs are contiguous)
    const int nout = rpb * NV;
    const int obb = tid / rpb, orr = tid - obb * rpb;
    half_t osv = (half_t)0.0f, osm = (half_t)0.0f;
    if (tid < nout) {
        osv = scale_vec[min(obb, batch - 1)];
        osm = scale_mat[min(row0 + orr, dim_out - 1)];
    }
#pragma unroll
    for (int g = 0; g < G; ++g) {
        int32_t acc[NV];
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            acc[v] = 0;
#pragma unroll
            for (int i = 0; i < PPL; ++i)
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[v] = __builtin_amdgcn_sdot4(wf[g][i][e], vf[v][i][e], acc[v], false);
        }
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int32_t t = wave_sum_i32_to_lane63(acc[v]);
            if (lane == 63) part[(g * 8 + w) * NV + v] = t;
        }
    }
    __syncthreads();
    if (tid < nout) {
        const int32_t row = row0 + orr;
        if (row < dim_out && obb < batch) out[(int64_t)obb * dim_out + row] = dequant(part[orr * NV + obb], (float)osv, (float)osm);
    }
}

// Generic path (any dim_in % 4 == 0, any alignment): one wave per matrix row, dword loads,
// v_dot4_i32_i8, up to 8 vectors per pass so the row is read from HBM once per 8 vectors.
__global__ __launch_bounds__(256) void k_gemv_dot4(int32_t batch, int32_t dim_out, int32_t dim_in,
                                                   const half_t* __restrict__ scale_mat,
                                                   const int8_t* __restrict__ mat,
                                                   const half_t* __restrict__ scale_vec,
                                                   const int8_t* __restrict__ vec,
                                                   half_t* __restrict__ out) {
    const int lane = threadIdx.x & 63;
    const int32_t row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= dim_out) return;
    const int32_t* mrow = reinterpret_cast<const int32_t*>(mat + (int64_t)row * dim_in);
    const int32_t k4 = dim_in >> 2;
    const float sm = (float)scale_mat[row];
    for (int32_t b0 = 0; b0 < batch; b0 += 8) {
        int32_t acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int32_t i = lane; i < k4; i += 64) {
            const int32_t wv = mrow[i];
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                if (b0 + t < batch) {
                    const int32_t vv = reinterpret_cast<const int32_t*>(vec + (int64_t)(b0 + t) * dim_in)[i];
                    acc[t] = __builtin_amdgcn_sdot4(wv, vv, acc[t], false);
                }
            }
        }
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const int32_t s = wave_sum_i32(acc[t]);
            if (lane == 0 && b0 + t < batch)
                out[(int64_t)(b0 + t) * dim_out + row] = dequant(s, (float)scale_vec[b0 + t], sm);
        }
    }
}

// Rows per workgroup, in steps of 4: one workgroup per compute unit when the matrix allows it
// (every workgroup re-reads all the vectors from L2, so fewer and larger ones are better), at
// most 16*MAXRG rows.
template <int NB, int MAXRG, bool F16 = false>
static void launch_coalesced(int32_t batch, int32_t dim_out, int32_t dim_in, const half_t* sm, const int8_t* mat,
                             const half_t* sv, const int8_t* vec, half_t* out, hipStream_t st) {
    int64_t r4 = ceil_div(ceil_div(dim_out, compute_units()), 4);
    if (r4 > 4 * MAXRG) r4 = 4 * MAXRG;
    if (r4 < 1) r4 = 1;
    const int rg = (int)ceil_div(r4, 4);
    const dim3 grid((unsigned)ceil_div(dim_out, r4 * 4));
    auto go = [&](auto rgc) {
        hipLaunchKernelGGL((k_gemv_coalesced<8, decltype(rgc)::value, NB, F16>), grid, dim3(512), 0, st, batch, dim_out, dim_in,
                           (int32_t)r4, sm, mat, sv, vec, out);
    };
    if constexpr (MAXRG >= 4) { if (rg == 4) return go(std::integral_constant<int, 4>{}); }
    if constexpr (MAXRG >= 3) { if (rg == 3) return go(std::integral_constant<int, 3>{}); }
    if constexpr (MAXRG >= 2) { if (rg == 2) return go(std::integral_constant<int, 2>{}); }
    go(std::integral_constant<int, 1>{});
}

// The row-wise kernel for one or two vectors: rows of 4 KB (up to 40 per compute unit) or 10 KB (up to 16 per
// compute unit) -- the row lengths of the model this path serves; at least two rows per wave, below that the
// matrix-core kernels are as quick.  ([10240, 4096] at one / two vectors: 7.8 / 8.5 us against 9.6 / 9.8 on the
// matrix cores; with three or four vectors the dot products and their sums over the wave cost what the access
// pattern saves.)
static bool launch_gemv_rowwise(int32_t batch, int32_t dim_out, int32_t dim_in, const half_t* sm, const int8_t* mat,
                                const half_t* sv, const int8_t* vec, half_t* out, hipStream_t st) {
    if (batch > 2 || (dim_in != 4096 && dim_in != 10240) || (int64_t)dim_out * dim_in >= (1ll << 32)) return false;
    const int nv = batch;
    const int64_t rpb = ceil_div(dim_out, compute_units());
    const int g = (int)ceil_div(rpb, 8);
    const dim3 grid((unsigned)ceil_div(dim_out, rpb));
    auto go = [&](auto kern) { hipLaunchKernelGGL(kern, grid, dim3(512), 0, st, batch, dim_out, (int32_t)rpb, sm, mat, sv, vec, out); };
    auto pick = [&](auto nvc, auto pplc) {
        constexpr int NV = decltype(nvc)::value, PPL = decltype(pplc)::value;
        if constexpr (PPL == 4) {
            if (g == 2) go(k_gemv_rowwise<NV, 4, 2>);
            else if (g == 3) go(k_gemv_rowwise<NV, 4, 3>);
            else if (g == 4) go(k_gemv_rowwise<NV, 4, 4>);
            else go(k_gemv_rowwise<NV, 4, 5>);
        } else {
            go(k_gemv_rowwise<NV, 10, 2>);
        }
    };
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I4 = std::integral_constant<int, 4>;
    if (dim_in == 4096 && g >= 2 && g <= 5) {
        if (nv == 1) pick(I1{}, I4{});
        else pick(I2{}, I4{});
        return true;
    }
    if (dim_in == 10240 && g == 2) {
        if (nv == 1) pick(I1{}, std::integral_constant<int, 10>{});
        else pick(I2{}, std::integral_constant<int, 10>{});
        return true;
    }
    return false;
}

template <int NB, bool DW = false>
static void launch_mfma(int32_t batch, int32_t dim_out, int32_t dim_in, const half_t* sm, const int8_t* mat,
                        const half_t* sv, const int8_t* vec, half_t* out, hipStream_t st) {
    // 32 rows per workgroup halves the L2 traffic for the vectors; keep 16 when that
    // would leave compute units without a workgroup.
    if (dim_out >= 32 * 256) {
        hipLaunchKernelGGL((k_gemv_mfma<8, 2, NB, DW>), dim3((unsigned)ceil_div(dim_out, 32)), dim3(512), 0, st,
                           batch, dim_out, dim_in, sm, mat, sv, vec, out);
    } else {
        hipLaunchKernelGGL((k_gemv_mfma<8, 1, NB, DW>), dim3((unsigned)ceil_div(dim_out, 16)), dim3(512), 0, st,
                           batch, dim_out, dim_in, sm, mat, sv, vec, out);
    }
}

// fp16 matrix with rows that are not whole 256-byte chunks, on the predicated MFMA kernel: rows of whole 16-byte pieces,
// or (DW) of whole dwords.  Returns -1 when the buffers are not aligned for it.
int gemv_f16_mfma(int32_t batch, int32_t dim_out, int32_t dim_in, const void* mat, const void* vec, void* out, hipStream_t st) {
    const int64_t row_bytes = (int64_t)dim_in * 2;
    if (dim_in <= 0 || row_bytes % 4 != 0 || row_bytes > 0x7fffffff || (reinterpret_cast<uintptr_t>(mat) & 3u) || (reinterpret_cast<uintptr_t>(vec) & 3u)) return -1;
    const bool dw = row_bytes % 16 != 0 || !aligned16(mat) || !aligned16(vec);
    const int8_t* M = (const int8_t*)mat;
    for (int32_t b0 = 0; b0 < batch; b0 += 32) {           // (the fp32 slices of 32 vectors x 32 rows x 8 waves fill 64 KB of LDS)
        const int32_t nb = batch - b0 < 32 ? batch - b0 : 32;
        const int8_t* v = (const int8_t*)vec + (int64_t)b0 * row_bytes;
        half_t* o = (half_t*)out + (int64_t)b0 * dim_out;
        auto go = [&](auto nbc, auto dwc) {
            constexpr int NB = decltype(nbc)::value;
            constexpr bool DW = decltype(dwc)::value;
            if (dim_out >= 32 * 256)
                hipLaunchKernelGGL((k_gemv_mfma<8, 2, NB, DW, true>), dim3((unsigned)ceil_div(dim_out, 32)), dim3(512), 0, st, nb, dim_out,
                                   (int32_t)row_bytes, nullptr, M, nullptr, v, o);
            else
                hipLaunchKernelGGL((k_gemv_mfma<8, 1, NB, DW, true>), dim3((unsigned)ceil_div(dim_out, 16)), dim3(512), 0, st, nb, dim_out,
                                   (int32_t)row_bytes, nullptr, M, nullptr, v, o);
        };
        using I1 = std::integral_constant<int, 1>;
        using I2 = std::integral_constant<int, 2>;
        if (nb <= 16) { if (dw) go(I1{}, std::true_type{}); else go(I1{}, std::false_type{}); }
        else { if (dw) go(I2{}, std::true_type{}); else go(I2{}, std::false_type{}); }
        if (int e = launch_status()) return e;
    }
    return 0;
}

// fp16 matrix (dim_out, dim_in) shared by `batch` fp16 vectors on the MFMA kernel above.  Returns -1 when
// the shape does not qualify (rows of whole 256-byte chunks, 16-byte aligned, offsets within 32 bits).
int gemv_f16_coalesced(int32_t batch, int32_t dim_out, int32_t dim_in, const void* mat, const void* vec, void* out, hipStream_t st) {
    const int64_t row_bytes = (int64_t)dim_in * 2;
    if (dim_in <= 0 || row_bytes % 256 != 0 || !aligned16(mat) || !aligned16(vec) || (int64_t)dim_out * row_bytes >= (1ll << 32))
        return -1;
    const int8_t* M = (const int8_t*)mat;
    for (int32_t b0 = 0; b0 < batch; b0 += 128) {
        const int32_t nb = batch - b0 < 128 ? batch - b0 : 128;
        if ((int64_t)nb * row_bytes >= (1ll << 32)) return -1;
        const int8_t* v = (const int8_t*)vec + (int64_t)b0 * row_bytes;
        half_t* o = (half_t*)out + (int64_t)b0 * dim_out;
        if (nb <= 16) launch_coalesced<1, 4, true>(nb, dim_out, (int32_t)row_bytes, nullptr, M, nullptr, v, o, st);
        else if (nb <= 32) launch_coalesced<2, 4, true>(nb, dim_out, (int32_t)row_bytes, nullptr, M, nullptr, v, o, st);
        else if (nb <= 64) launch_coalesced<4, 2, true>(nb, dim_out, (int32_t)row_bytes, nullptr, M, nullptr, v, o, st);
        else launch_coalesced<8, 1, true>(nb, dim_out, (int32_t)row_bytes, nullptr, M, nullptr, v, o, st);
        if (int e = launch_status()) return e;
    }
    return 0;
}

}  // namespace cpmk

using namespace cpmk;

extern "C" int cpmk_gemv_broadcast_mat_int8(int32_t batch, int32_t dim_out, int32_t dim_in,
                                            const void* scale_mat, const void* mat, const void* scale_vec,
                                            const void* vec, void* out, void* stream) {
    clear_stale_error();
    if (batch < 0 || dim_out < 0 || dim_in < 0) return CPMK_EBADARG;
    if (dim_in % 4) return CPMK_EALIGN;   // kernels/gemv.py:65
    if (batch == 0 || dim_out == 0) return 0;
    if (any_null(scale_mat, scale_vec, out) || (dim_in > 0 && any_null(mat, vec))) return CPMK_EBADARG;
    hipStream_t st = (hipStream_t)stream;
    const half_t* sm = (const half_t*)scale_mat;
    const half_t* sv = (const half_t*)scale_vec;
    const int8_t* M = (const int8_t*)mat;
    const int8_t* V = (const int8_t*)vec;
    half_t* O = (half_t*)out;
    const bool fast = dim_in > 0 && (dim_in % 16 == 0) && aligned16(mat) && aligned16(vec);
    if (!fast) {
        if (dim_in > 0 && (reinterpret_cast<uintptr_t>(mat) & 3u) == 0 && (reinterpret_cast<uintptr_t>(vec) & 3u) == 0) {
            // rows that are only 4-byte aligned (dim_in % 16 != 0, e.g. the 8888 of the reference's tests/test_gemv.py:12):
            // the matrix-core kernel on 4-byte loads, up to 128 vectors per pass over the matrix
            for (int32_t b0 = 0; b0 < batch; b0 += 128) {
                const int32_t nb = batch - b0 < 128 ? batch - b0 : 128;
                const int8_t* v = V + (int64_t)b0 * dim_in;
                half_t* o = O + (int64_t)b0 * dim_out;
                if (nb <= 16) launch_mfma<1, true>(nb, dim_out, dim_in, sm, M, sv + b0, v, o, st);
                else if (nb <= 32) launch_mfma<2, true>(nb, dim_out, dim_in, sm, M, sv + b0, v, o, st);
                else if (nb <= 64) launch_mfma<4, true>(nb, dim_out, dim_in, sm, M, sv + b0, v, o, st);
                else launch_mfma<8, true>(nb, dim_out, dim_in, sm, M, sv + b0, v, o, st);
                if (int e = launch_status()) return e;
            }
            return 0;
        }
        hipLaunchKernelGGL(k_gemv_dot4, dim3((unsigned)ceil_div(dim_out, 4)), dim3(256), 0, st, batch, dim_out,
                           dim_in, sm, M, sv, V, O);
        return launch_status();
    }
    // up to 128 vectors per pass over the matrix
    for (int32_t b0 = 0; b0 < batch; b0 += 128) {
        const int32_t nb = batch - b0 < 128 ? batch - b0 : 128;
        const int8_t* v = V + (int64_t)b0 * dim_in;
        half_t* o = O + (int64_t)b0 * dim_out;
        const half_t* s = sv + b0;
        if (launch_gemv_rowwise(nb, dim_out, dim_in, sm, M, s, v, o, st)) {
        } else if (dim_in % 256 == 0 && (int64_t)dim_out * dim_in < (1ll << 32) && (int64_t)nb * dim_in < (1ll << 32)) {
            if (nb <= 16) launch_coalesced<1, 4>(nb, dim_out, dim_in, sm, M, s, v, o, st);
            else if (nb <= 32) launch_coalesced<2, 4>(nb, dim_out, dim_in, sm, M, s, v, o, st);
            else if (nb <= 64) launch_coalesced<4, 2>(nb, dim_out, dim_in, sm, M, s, v, o, st);
            else launch_coalesced<8, 1>(nb, dim_out, dim_in, sm, M, s, v, o, st);
        } else if (nb <= 16) launch_mfma<1>(nb, dim_out, dim_in, sm, M, s, v, o, st);
        else if (nb <= 32) launch_mfma<2>(nb, dim_out, dim_in, sm, M, s, v, o, st);
        else if (nb <= 64) launch_mfma<4>(nb, dim_out, dim_in, sm, M, s, v, o, st);
        else launch_mfma<8>(nb, dim_out, dim_in, sm, M, s, v, o, st);
        if (int e = launch_status()) return e;
    }
    return 0;
}
