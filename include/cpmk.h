/*
 * cpmk.h -- C ABI of libcpmk_hip.so: hand-written HIP kernels for gfx950 (MI355X) that
 * implement the int8 quantized-GEMM inference path of OpenBMB/cpm_kernels.
 *
 * Conventions
 *   - Every pointer is a raw device address on the current HIP device; the caller owns
 *     all buffers (inputs, outputs); nothing is allocated per call.
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *   - Every launcher is asynchronous and returns 0 on success, a hipError_t value if the
 *     HIP runtime reported an error at launch, or a CPMK_E* code (>= 10000) for an
 *     argument the kernels cannot handle.  cpmk_error_string() explains any of them.
 *   - Launch geometry is private to the library (the reference computes grid/block in
 *     its Python wrappers; here the Python wrappers only forward arguments).
 *   - fp16 is IEEE binary16; "b,n,m" tensors are row-major with m contiguous.
 *
 * Each declaration cites the reference interface it replaces as
 * <python wrapper file:line> / <CUDA kernel file:line> relative to the reference tree.
 */
#ifndef CPMK_H_
#define CPMK_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CPMK_EBADARG   10001  /* negative size, null pointer with non-empty work, ...   */
#define CPMK_EALIGN    10002  /* divisibility precondition of the reference violated    */
#define CPMK_ETOOBIG   10003  /* problem exceeds a documented limit of this library     */

/* ---- library / device queries (replace cpm_kernels/library/cudart.py and
 *      cpm_kernels/device/__init__.py:106-158) ------------------------------------ */
int         cpmk_version(void);                       /* e.g. 10000 = 1.0.0 */
const char* cpmk_error_string(int code);
int         cpmk_device_count(int* count);            /* cudart.cudaGetDeviceCount  */
int         cpmk_get_device(int* device);             /* cudart.cudaGetDevice       */
int         cpmk_set_device(int device);              /* cudart.cudaSetDevice       */
/* Fills name (NUL-terminated, e.g. "gfx950"), compute units, LDS bytes per workgroup,
 * wavefront size, max engine clock in kHz, memory clock in kHz, memory bus width in
 * bits, L2 bytes, total global memory bytes.  Any out pointer may be NULL.
 * (device/__init__.py:106-113 caches 101 cudaDevAttr* values; these are the ones the
 * path and its roofline need.) */
int         cpmk_device_props(int device, char* name, int name_len, int* compute_units,
                              int* lds_bytes, int* wavefront, int* clock_khz,
                              int* mem_clock_khz, int* mem_bus_bits, int* l2_bytes,
                              uint64_t* global_mem_bytes);

/* ---- row / column quantisation (kernels/gemm.py, cuda/gemm.cu) ------------------- */
/* out[b,i] = fp16( max_j |mat[b,i,j]| / 127 )            gemm.py:91-107 / gemm.cu:60-76 */
int cpmk_gemm_calc_scale(int32_t batch, int32_t n, int32_t m,
                         const void* mat /* (b,n,m) fp16 */, void* out /* (b,n) fp16 */,
                         void* stream);
/* out[b,j] = fp16( max_i |mat[b,i,j]| / 127 )           gemm.py:109-125 / gemm.cu:79-98 */
int cpmk_gemm_calc_scale_transpose(int32_t batch, int32_t n, int32_t m,
                                   const void* mat /* (b,n,m) fp16 */,
                                   void* out /* (b,m) fp16 */, void* stream);
/* out[b,i,j] = int8( rint( f32(mat[b,i,j]) / f32(scale[b,i]) ) )
 *                                                        gemm.py:21-41 / gemm.cu:6-18 */
int cpmk_gemm_round(int32_t batch, int32_t n, int32_t m,
                    const void* mat /* (b,n,m) fp16 */, const void* scale /* (b,n) fp16 */,
                    void* out /* (b,n,m) int8 */, void* stream);
/* out[b,i,j] = int8( rint( f32(mat[b,i,j]) / f32(scale[b,j]) ) )
 *                                                        gemm.py:43-63 / gemm.cu:22-33 */
int cpmk_gemm_round_transpose(int32_t batch, int32_t n, int32_t m,
                              const void* mat, const void* scale /* (b,m) fp16 */,
                              void* out, void* stream);
/* out[b,i,j] = fp16( (f32(mat[b,i,j]) * sx) * f32(sy[j]) ),
 * sx = scale_x[broad_cast_x ? i : b*n+i], sy = scale_y + (broad_cast_y ? 0 : b*m)
 *                                                        gemm.py:65-89 / gemm.cu:37-57 */
int cpmk_gemm_scale(int32_t batch, int32_t n, int32_t m,
                    const void* mat /* (b,n,m) int32 */, const void* scale_x /* fp16 */,
                    const void* scale_y /* fp16 */, void* out /* (b,n,m) fp16 */,
                    int broad_cast_x, int broad_cast_y, void* stream);
/* out = fp16( f32(scale_x[b,i]) * f32(mat) )           gemm.py:309-327 / gemm.cu:176-189 */
int cpmk_gemm_scale_x(int32_t batch, int32_t n, int32_t m, const void* mat,
                      const void* scale_x /* (b,n) fp16 */, void* out, void* stream);
/* out = fp16( f32(mat) * f32(scale_y[b,j]) )           gemm.py:329-347 / gemm.cu:192-205 */
int cpmk_gemm_scale_y(int32_t batch, int32_t n, int32_t m, const void* mat,
                      const void* scale_y /* (b,m) fp16 */, void* out, void* stream);

/* ---- int8 x int8 -> int32 batched GEMM (replaces the cuBLASLt call in
 *      kernels/gemm.py:127-186 and library/cublaslt.py:113-150) --------------------
 * out[b,j,i] = sum_kk A'[b,kk,i] * B'[b,j,kk]   for i < m, j < n, kk < k, where
 *   A is stored row-major (k,m) if !aT, (m,k) if aT;
 *   B is stored row-major (n,k) if !bT, (k,n) if bT;
 *   out is row-major (max(batchA,batchB), n, m) int32;
 *   an operand whose batch is 1 is broadcast (batch stride 0).
 * Preconditions of the reference kept: m,k,n multiples of 4 (CPMK_EALIGN otherwise),
 * batchA == batchB or one of them 1 (CPMK_EBADARG otherwise). */
int cpmk_gemm_int8(int32_t m, int32_t k, int32_t n, int32_t batchA, int32_t batchB,
                   int aT, int bT, const void* A, const void* B, void* out, void* stream);

/* Same product with the dequantising epilogue of cpmk_gemm_scale applied to the int32
 * accumulators in registers, writing fp16 (max(batchA,batchB), n, m):
 *   out[b,j,i] = fp16( (f32(acc) * f32(scale_row[bcr ? j : b*n+j])) * f32(scale_col[(bcc ? 0 : b*m) + i]) )
 * Bit-identical to cpmk_gemm_int8 followed by cpmk_gemm_scale; it fuses what
 * cpm_kernels/torch/gemm.py:40-64 (gemm_and_scale) does in two launches and one int32
 * round trip through memory. */
int cpmk_gemm_int8_scale(int32_t m, int32_t k, int32_t n, int32_t batchA, int32_t batchB,
                         int aT, int bT, const void* A, const void* B,
                         const void* scale_row /* fp16, per out row j */,
                         const void* scale_col /* fp16, per out col i */,
                         int broad_cast_row, int broad_cast_col,
                         void* out /* fp16 */, void* stream);

/* Fused absmax + round of cpm_kernels/torch/gemm.py:5-38 (calc_scale then round_i8 on the
 * same tensor): one read of mat, writes scale and the int8 tensor.  transpose = 0 uses
 * per-row scales (b,n); transpose = 1 per-column scales (b,m).  Bit-identical to the two
 * separate launchers. */
int cpmk_gemm_quantize(int32_t batch, int32_t n, int32_t m, const void* mat,
                       void* scale, void* out, int transpose, void* stream);

/* cpmk_gemm_quantize(transpose = 0) of two tensors with rows of the same length m in one
 * launch: rows0 x m at mat0 and rows1 x m at mat1 (batch and row dimensions flattened), each
 * with its own scale and int8 output.  What torch-level bmm needs for its two operands; no
 * counterpart in the reference. */
int cpmk_gemm_quantize_pair(int64_t rows0, const void* mat0, void* scale0, void* out0,
                            int64_t rows1, const void* mat1, void* scale1, void* out1,
                            int32_t m, void* stream);

/* Per-column scales (b,m) and rounding in one pass, as cpmk_gemm_quantize with transpose = 1
 * (cpm_kernels/torch/gemm.py:98-102 for an operand given as (b, K, N)), with the int8 result
 * written in place (b,n,m) when out_transposed = 0 or transposed (b,m,n) when 1.  The transposed
 * form has no counterpart in the reference, where cuBLASLt consumes the operand as it lies; here
 * it turns such an operand into the K-major layout of the fast int8 GEMM.  Values are
 * bit-identical to calc_scale_transpose + round_transpose. */
int cpmk_gemm_quantize_cols(int32_t batch, int32_t n, int32_t m, const void* mat,
                            void* scale, void* out, int out_transposed, void* stream);

/* ---- fp16 products next to the path (attention scores, fp16 decode) ---------------- */
/* Same operand convention as cpmk_gemm_int8 with fp16 operands and fp16 output, fp32
 * accumulation (the reference asks cuBLASLt for fp16 accumulation where the device has it).
 * Requires m, n, k even as the reference asserts.        kernels/gemm.py:188-256 (cuBLASLt) */
int cpmk_gemm_fp16(int32_t m, int32_t k, int32_t n, int32_t batchA, int32_t batchB,
                   int aT, int bT, const void* A, const void* B, void* out, void* stream);
/* out[b,o] = sum_k mat[b,o,k] vec[b,k]      kernels/gemv.py:82-149 / cuda/gemv.cu:78-107 */
int cpmk_gemv_fp16(int32_t batch, int32_t dim_out, int32_t dim_in, const void* mat,
                   const void* vec, void* out, void* stream);
/* out[b,o] = sum_k mat[b,k,o] vec[b,k]      kernels/gemv.py:151-216 / cuda/gemv.cu:109-140 */
int cpmk_gemv_fp16_transpose(int32_t batch, int32_t dim_out, int32_t dim_in, const void* mat,
                             const void* vec, void* out, void* stream);
/* out[b,o] = sum_k mat[o,k] vec[b,k]        kernels/gemv.py:218-283 / cuda/gemv.cu:142-175 */
int cpmk_gemv_broadcast_mat_fp16(int32_t batch, int32_t dim_out, int32_t dim_in, const void* mat,
                                 const void* vec, void* out, void* stream);

/* ---- callers either side of the path in a decode loop ----------------------------- */
/* out[b,i,j] = weights[ids[b,j], i];  ids (b, seq) int32, weights (vocab, hidden) fp16,
 * out (b, hidden, seq) fp16                    kernels/embedding.py:14-34 / embedding.cu:6-37 */
int cpmk_embedding_forward(int32_t batch, int32_t hidden_size, int32_t seq_len, const void* ids,
                           const void* weights, void* out, void* stream);
/* out[b,:] = weights[ids[b],:]                 kernels/embedding.py:88-105 / embedding.cu:90-103 */
int cpmk_embedding_step(int32_t batch, int32_t embedding_size, const void* ids,
                        const void* weights, void* out, void* stream);
/* out[b,pos,:] = inp[b,:];  out (b, buffer_len, n) fp16, n % 2 == 0
 *                                              kernels/utils.py:18-37 / utils.cu:13-29 */
int cpmk_copy_data_to_kv(int32_t batch, int32_t buffer_len, int32_t n, const void* inp,
                         void* out, int32_t pos, void* stream);

/* ---- decode GEMV (kernels/gemv.py, cuda/gemv.cu) --------------------------------- */
/* out[b] = fp16( max_j |vec[b,j]| / 127 )                gemv.py:18-33 / gemv.cu:26-40 */
int cpmk_gemv_calc_scale(int32_t batch, int32_t n, const void* vec, void* out, void* stream);
/* out[b,j] = int8( rint( f32(vec[b,j]) / f32(scale[b]) ) )  gemv.py:35-53 / gemv.cu:43-54 */
int cpmk_gemv_round(int32_t batch, int32_t n, const void* vec, const void* scale,
                    void* out, void* stream);
/* out[b,o] = fp16( (f32(sum_k mat[o,k]*vec[b,k]) * f32(scale_vec[b])) * f32(scale_mat[o]) )
 * dim_in % 4 == 0 (CPMK_EALIGN otherwise).             gemv.py:56-79 / gemv.cu:57-76 */
int cpmk_gemv_broadcast_mat_int8(int32_t batch, int32_t dim_out, int32_t dim_in,
                                 const void* scale_mat /* (dim_out) fp16 */,
                                 const void* mat /* (dim_out,dim_in) int8 */,
                                 const void* scale_vec /* (batch) fp16 */,
                                 const void* vec /* (batch,dim_in) int8 */,
                                 void* out /* (batch,dim_out) fp16 */, void* stream);

/* ---- normalisation over dim 1 of (batch,n,m) (kernels/layernorm.py, cuda/layernorm.cu)
 * mean = rd_mean ? sum_i x/n : 0;  var = sum_i x^2/n - mean^2;
 * out = fp16( (x - mean) * rsqrt(var + eps) ).  out may alias mat.
 *                         layernorm.py:18-58 / layernorm.cu:6-71 (inplace: :75-139) */
int cpmk_layernorm_forward(int32_t batch, int32_t n, int32_t m, const void* mat, void* out,
                           float eps, int rd_mean, void* stream);
/* Same normalisation over the contiguous last dim of (batch,n) (the decode-step form).
 *                         layernorm.py:152-190 / layernorm.cu:343-421 */
int cpmk_layernorm_step(int32_t batch, int32_t n, const void* mat, void* out, float eps,
                        int rd_mean, void* stream);
/* Normalisation followed by the affine of arith_ln_mul_add / arith_ln_mul applied to the
 * fp16-rounded result (beta == NULL -> multiply only), as
 * cpm_kernels/torch/layernorm.py:9-29,88-111 do in two launches.  Bit-identical to them. */
int cpmk_layernorm_affine_forward(int32_t batch, int32_t n, int32_t m, const void* mat,
                                  const void* alpha /* (n) fp16 */,
                                  const void* beta /* (n) fp16 or NULL */, void* out,
                                  float eps, int rd_mean, void* stream);

/* ---- softmax over dim 1 of (batch,n,m) (kernels/softmax.py, cuda/softmax.cu) ------
 * M = max(max_i x, -1e6); S = sum_i exp(x-M) + 1e-10; out = fp16(exp(x-M)/S).
 * out may alias inp.        softmax.py:14-46 / softmax.cu:6-43 (inplace: :46-82) */
int cpmk_softmax_forward(int32_t batch, int32_t n, int32_t m, const void* inp, void* out,
                         void* stream);
/* Same over the contiguous last dim of (batch,n), in place.
 *                           softmax.py:68-81 / softmax.cu:117-159 */
int cpmk_softmax_step_inplace(int32_t batch, int32_t n, void* x, void* stream);

/* ---- GELU (kernels/gelu.py:13-48, cuda/gelu.cu:6-17) ------------------------------
 * out = fp16( 0.5*x*(1 + tanhf(0.7978845608028654*x*(1 + 0.044715*x*x))) ), out may alias mat */
int cpmk_gelu_forward(int32_t batch, int32_t n, const void* mat, void* out, void* stream);

/* ---- relative position bias (kernels/position_bucket.py, cuda/position_bucket.cu) -- */
/* int32 bucket table of max_distance entries.  position_bucket.py:14-30 / .cu:6-21 */
int cpmk_position_embedding_init(int32_t num_buckets, int32_t max_distance, void* out,
                                 int bidirectional, void* stream);
/* out[h,k,q] = weight[h, table[rel] + off]            position_bucket.py:32-58 / .cu:25-54 */
int cpmk_position_embedding_forward(int32_t query_len, int32_t key_len, int32_t num_buckets,
                                    int32_t max_distance, int32_t num_heads,
                                    const void* position_mapping /* int32 */,
                                    const void* weight /* (heads,buckets) fp16 */,
                                    void* out /* (heads,key_len,query_len) fp16 */,
                                    int bidirectional, void* stream);
/* out[h,k] for a single query position.               position_bucket.py:88-113 / .cu:105-133 */
int cpmk_position_embedding_step(int32_t query_pos, int32_t key_len, int32_t num_buckets,
                                 int32_t max_distance, int32_t num_heads,
                                 const void* position_mapping, const void* weight,
                                 void* out /* (heads,key_len) fp16 */, int bidirectional,
                                 void* stream);

/* ---- elementwise helpers used by the path's callers ------------------------------ */
/* out = fp16_fma(x, alpha[n], beta[n]); m % 2 == 0.   kernels/arith.py:135-161 / arith.cu:97-112 */
int cpmk_arith_ln_mul_add(int32_t batch, int32_t n, int32_t m, const void* inp,
                          const void* alpha, const void* beta, void* out, void* stream);
/* out = x * alpha[n] (fp16); m % 2 == 0.              kernels/arith.py:190-214 / arith.cu:115-127 */
int cpmk_arith_ln_mul(int32_t batch, int32_t n, int32_t m, const void* inp,
                      const void* alpha, void* out, void* stream);
/* out = x + y (fp16); n % 2 == 0.                     kernels/arith.py:43-66 / arith.cu:19-30 */
int cpmk_arith_element_add(int32_t batch, int32_t n, const void* x, const void* y,
                           void* out, void* stream);
/* out[b,i,j] = mask[b,j] == 0 ? fp16(value) : x[b,i,j]    kernels/mask.py:12-35 / mask.cu:6-23 */
int cpmk_mask(int32_t batch, int32_t n, int32_t m, const void* inp,
              const void* mask /* (b,m) int8 */, float value, void* out, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* CPMK_H_ */
