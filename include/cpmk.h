/*
 * cpmk.h -- C ABI of libcpmk_hip.so: hand-written HIP kernels for gfx950 (MI355X) that
 * implement the int8 quantized-GEMM inference path of OpenBMB/cpm_kernels.
 *
 * Conventions
 *   - Every pointer is a raw device address on the current HIP device; the caller owns
 *     all buffers (inputs, outputs); nothing is allocated per call.
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *   - Every launcher is asynchronous and returns 0 on success, a hipError_t value if the
 *     HIP runtime reported an error at launch, a CPMK_E* code (>= 10000) for an
 *     argument the kernels cannot handle, or CPMK_ETIMEOUT while a failure of an earlier
 *     kernel is pending (cpmk_async_status).  cpmk_error_string() explains any of them.
 *   - Launch geometry is private to the library (the reference computes grid/block in
 *     its Python wrappers; here the Python wrappers only forward arguments).
 *   - fp16 is IEEE binary16; "b,n,m" tensors are row-major with m contiguous.
 *   - Sizes: element counts and byte offsets are 64-bit throughout (tensors beyond 2^31
 *     elements work), and batches of any int32 size are split over launches where a kernel
 *     indexes the batch with a grid dimension.  CPMK_ETOOBIG remains for: a matrix dimension
 *     beyond 4 194 240 (65535 tiles of 64) in the transposes and the embedding kernels; k above
 *     2^30 in the fp16 GEMM; more than 524 280 vectors in the general fp16 broadcast GEMV; more
 *     than 2^31-1 rows in the elementwise and row-quantising training kernels; more than 8192
 *     buckets in the position-bias gradient.
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
#define CPMK_ETIMEOUT  10004  /* a kernel's bounded wait ran out (sticky, see cpmk_async_status) */

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

/* Failures that a kernel can only discover while it runs.  The kernels that split a column over
 * several workgroups (tall layernorm / softmax, the column quantiser, the dim-1 reductions of the
 * training side) wait for each other's partial results with a bound of about one second; a wait
 * that runs out fills the affected outputs with NaN (0 in int8 tensors) and sets a sticky word on
 * the device and its mirror in pinned host memory.  From then on EVERY launcher of this library
 * returns CPMK_ETIMEOUT instead of 0 (its own launch is still made), so the failure is reported by
 * the next call on that device, whichever it is, as the reference reports every failure of a launch
 * or a synchronisation from its status checks (library/cudart.py:325-327, cudaGetLastError); the
 * Python binding raises RuntimeError on any non-zero status.  cpmk_async_status() returns the
 * condition (0, CPMK_ETIMEOUT, or a HIP error code) and clears it; it runs a one-thread kernel on
 * the null stream and blocks like a hipMemcpy, so it also catches a time-out of work that has only
 * just finished: synchronise the streams in question first, then call it (a serving loop: once per
 * step, where it synchronises anyway). */
int         cpmk_async_status(void);
/* Launches one workgroup that waits `microseconds` for a result nobody produces and then reports
 * the time-out as above: exercises the failure path with a kernel that ends normally (tests). */
int         cpmk_selftest_exchange_timeout(int32_t microseconds, void* stream);
/* A team launch recorded during stream capture is given packet slots that stay with its graph for good
 * (it may be replayed at any time), out of a reserve of 32768 per device; a tall layernorm of
 * 8 x 4096 x 512 takes 256, and the launches recorded on one stream during one capture, which run one
 * after the other, share the slots of the largest of them.  Writes how many are left on the current
 * device.  When a recorded call needs more than are left, the library records kernels that need no
 * packets instead (same results for the exact kernels, the same tolerances for layernorm and
 * softmax, more time). */
int         cpmk_exchange_capture_slots_left(int32_t* slots);

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
/* cpmk_layernorm_forward for callers that cannot let the library allocate or track anything: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc and event creation.
 * It has no counterpart in the reference.  Same arguments, same results to the bit.  Columns taller
 * than 1024 rows are normalised by teams of workgroups that exchange partial sums through a fixed
 * 2.1 MB array inside the library (2048 packet slots, one per (64-column tile, row part) pair; held
 * by every GPU the library runs on) instead of the shared pool with its completion events: a call
 * that needs more slots -- batch * ceil(m/64) * ceil(n / R) > 2048, where R is the rows per part that
 * cpmk_layernorm_forward uses for the shape: 1024 for n > 4096, and for n >= 2048 when
 * batch * ceil(m/64) * ceil(n/1024) does not exceed the number of compute units, else 512 -- returns
 * CPMK_ETOOBIG.  Makes no hipMalloc/hipFree/event call.  Every call on a GPU uses that GPU's one
 * array: calls that overlap in time on one GPU (two streams, two host threads, a replay of a
 * captured call concurrent with another) race; calls in stream order are safe. */
int cpmk_layernorm_forward_noalloc(int32_t batch, int32_t n, int32_t m, const void* mat, void* out,
                                   float eps, int rd_mean, void* stream);
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

/* ---- training side and remaining helpers of the kernels layer ---------------------------------
 * Not on the inference hot path; same arithmetic as the reference (fp16 ops round once, sums
 * accumulate in fp32; the order of fp32 summation differs, so sums agree to rounding only). */

/* out = fp16(float(x) * scale) over n elements; n % 2 == 0 asserted by the reference wrapper.
 *                                                     kernels/arith.py:24-41 / arith.cu:6-16 */
int cpmk_arith_global_scale(int64_t n, const void* inp, float scale, void* out, void* stream);
/* out = x * y (fp16); n % 2 == 0.                     kernels/arith.py:68-91 / arith.cu:33-44 */
int cpmk_arith_element_mul(int32_t batch, int32_t n, const void* x, const void* y, void* out, void* stream);
/* out[b,j] = x[b,j] + y[j]; n % 2 == 0.               kernels/arith.py:93-116 / arith.cu:47-58 */
int cpmk_arith_batch_add_forward(int32_t batch, int32_t n, const void* x, const void* y, void* out, void* stream);
/* grad[j] = sum_b grad_out[b,j].                      kernels/arith.py:118-133 / arith.cu:61-77 */
int cpmk_arith_batch_add_backward(int32_t batch, int32_t n, const void* grad_out, void* grad, void* stream);
/* out[b,i,j] = x[b,i,j] + beta[i]; m % 2 == 0.        kernels/arith.py:163-188 / arith.cu:80-94 */
int cpmk_arith_ln_add(int32_t batch, int32_t n, int32_t m, const void* inp, const void* beta, void* out, void* stream);
/* out[b,i,j] = x * fp16(1 / alpha[i]); m % 2 == 0.    kernels/arith.py:216-240 / arith.cu:131-143 */
int cpmk_arith_ln_div(int32_t batch, int32_t n, int32_t m, const void* inp, const void* alpha, void* out, void* stream);
/* out = fp16_fma(x, fp16(1/alpha[i]), fp16(-beta[i]/alpha[i])); m % 2 == 0.
 *                                                     kernels/arith.py:242-269 / arith.cu:146-165 */
int cpmk_arith_ln_sub_div(int32_t batch, int32_t n, int32_t m, const void* inp, const void* alpha, const void* beta,
                          void* out, void* stream);
/* grad[i] = sum_{b,j} x[b,i,j] * grad_out[b,i,j].     kernels/arith.py:271-289 / arith.cu:168-214 */
int cpmk_arith_ln_mul_backward(int32_t batch, int32_t n, int32_t m, const void* inp, const void* grad_out, void* grad,
                               void* stream);
/* grad[i] = sum_{b,j} grad_out[b,i,j].                kernels/arith.py:291-307 / arith.cu:217-261 */
int cpmk_arith_ln_add_backward(int32_t batch, int32_t n, int32_t m, const void* grad_out, void* grad, void* stream);
/* out[b,j] = fp16_fma(x[b,j], alpha[j], beta[j]); n % 2 == 0.   kernels/arith.py:309-331 / arith.cu:264-275 */
int cpmk_arith_batch_mul_add(int32_t batch, int32_t n, const void* x, const void* alpha, const void* beta, void* out,
                             void* stream);
/* out[b,j] = x[b,j] * alpha[j]; n % 2 == 0.           kernels/arith.py:333-354 / arith.cu:278-288 */
int cpmk_arith_batch_mul(int32_t batch, int32_t n, const void* x, const void* alpha, void* out, void* stream);

/* grad = gelu'(mat) * grad_out (tanh form, derivative 0/1 outside |x| < 5).
 *                                                     kernels/gelu.py:50-69 / gelu.cu:20-45 */
int cpmk_gelu_backward(int32_t batch, int32_t n, const void* grad_out, const void* mat, void* grad, void* stream);

/* grad[b,i,j] = out[b,i,j] * (grad_out[b,i,j] - sum_i out*grad_out).   kernels/softmax.py:48-66 / softmax.cu:86-114 */
int cpmk_softmax_backward(int32_t batch, int32_t n, int32_t m, const void* out, const void* grad_out, void* grad,
                          void* stream);

/* RMS-norm over dim 1 that also returns out_var[b,j] = rsqrt(mean(x^2) + eps) as fp16.
 *                                                     kernels/layernorm.py:60-80 / layernorm.cu:142-184 */
int cpmk_layernorm_forward_v(int32_t batch, int32_t n, int32_t m, const void* mat, void* out, void* out_var, float eps,
                             void* stream);
/* Mean-subtracting norm that also returns out_mean and out_var (reciprocal std), both (batch, m) fp16.
 *                                                     kernels/layernorm.py:82-104 / layernorm.cu:187-241 */
int cpmk_layernorm_forward_mv(int32_t batch, int32_t n, int32_t m, const void* mat, void* out, void* out_mean,
                              void* out_var, float eps, void* stream);
/* Gradient of forward_v given its out_var.            kernels/layernorm.py:106-126 / layernorm.cu:244-282 */
int cpmk_layernorm_backward_v(int32_t batch, int32_t n, int32_t m, const void* mat, const void* grad_out,
                              const void* var, void* grad, void* stream);
/* Gradient of forward_mv given its out_mean/out_var.  kernels/layernorm.py:128-150 / layernorm.cu:285-339 */
int cpmk_layernorm_backward_mv(int32_t batch, int32_t n, int32_t m, const void* mat, const void* grad_out,
                               const void* mean, const void* var, void* grad, void* stream);

/* scale_x[b,i] = max_j |mat*scale_y| / 127 (fp16 out), out = int8(rint(mat*scale_y / that quotient in fp32)).
 *                                                     kernels/gemm.py:261-283 / gemm.cu:102-133 */
int cpmk_gemm_backward_round_scale(int32_t batch, int32_t n, int32_t m, const void* mat, const void* scale_y,
                                   void* out, void* scale_x, int broad_cast_y, void* stream);
/* The same along dim 1: scale_y[b,j] from max_i |mat*scale_x|.   kernels/gemm.py:285-307 / gemm.cu:136-172 */
int cpmk_gemm_backward_scale_round(int32_t batch, int32_t n, int32_t m, const void* mat, const void* scale_x,
                                   void* out, void* scale_y, int broad_cast_x, void* stream);

/* grad[h, bucket] = sum of grad_out[h,k,q] over the (k,q) of the bucket; num_buckets <= 8192.
 *                                                     kernels/position_bucket.py:60-86 / position_bucket.cu:57-103 */
int cpmk_position_embedding_backward(int32_t query_len, int32_t key_len, int32_t num_buckets, int32_t max_distance,
                                     int32_t num_heads, const void* position_mapping, const void* grad_out,
                                     void* grad, int bidirectional, void* stream);

/* Embedding gradient, stage 1: per batch entry, runs of equal sorted ids summed; complete runs to grad,
 * the last run to aux_grad/aux_grad_idx.              kernels/embedding.py:36-65 / embedding.cu:36-64 */
int cpmk_embedding_backward_stage1(int32_t batch, int32_t seq_len, int32_t hidden_size, const void* grad_out,
                                   const void* argsort_ids, const void* sorted_ids, void* grad, void* aux_grad,
                                   void* aux_grad_idx, void* stream);
/* Stage 2: aux rows added into grad, equal neighbours merged first.   kernels/embedding.py:67-86 / embedding.cu:67-88 */
int cpmk_embedding_backward_stage2(int32_t batch, int32_t hidden_size, const void* aux_grad, const void* aux_grad_idx,
                                   void* grad, void* stream);

/* (batch, n, m) -> (batch, m, n), fp16.               kernels/transpose.py:11-29 / transpose.cu:6-24 */
int cpmk_transpose(int32_t batch, int32_t n, int32_t m, const void* inp, void* out, void* stream);

/* (batch, n, m) -> (batch, m, n), int8.  No counterpart in the reference, whose cuBLASLt call takes
 * int8 operands in either layout (kernels/gemm.py:127-186): the backward products of
 * torch/gemm.py:115-186 use this to bring their operands to the layout of the MFMA tile kernel. */
int cpmk_transpose_i8(int32_t batch, int32_t n, int32_t m, const void* inp, void* out, void* stream);
/* array[pos] += val (int32).                          kernels/utils.py:39-53 / utils.cu:31-35 */
int cpmk_array_add(void* array, int32_t pos, int32_t val, void* stream);
/* logits = logits / temperature - frequency_penalty*freq - presence_penalty*(freq > 0), in place.
 *                                                     kernels/utils.py:55-77 / utils.cu:38-54 */
int cpmk_adjustify_logits(int32_t batch, int32_t n, void* logits, float temperature, float frequency_penalty,
                          float presence_penalty, const void* frequency, void* stream);
/* new[b, :old_size] = old[b, :]; the rest of new untouched.   kernels/utils.py:79-96 / utils.cu:57-67 */
int cpmk_copy_extend_buffer(int32_t batch, int32_t old_size, int32_t nw_size, const void* old_buffer,
                            void* new_buffer, void* stream);
/* out[0] = 1 if any fp16 of inp is inf or NaN, otherwise out is left as it was.
 *                                                     kernels/utils.py:98-112 / utils.cu:70-88 */
int cpmk_has_nan_inf(int64_t n, const void* inp, void* out, void* stream);
/* out[b,h] = inp[b,h,pos] for inp (batch, hidden, seq_len).   kernels/utils.py:114-134 / utils.cu:91-101 */
int cpmk_copy_pos_hidden(int32_t batch, int32_t hidden_size, int32_t seq_len, int32_t pos, const void* inp,
                         void* out, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* CPMK_H_ */
