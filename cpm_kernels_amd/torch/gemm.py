"""``bmm(A, aT, B, bT, int8)`` with the interface of cpm_kernels/torch/gemm.py:233-239.

int8=True is the hot path: row-wise absmax quantisation of both operands, int8 GEMM with
int32 accumulation, fp16 dequantisation (GEMMInt8.forward, torch/gemm.py:84-113).  The
reference does that in six launches with an int32 round trip; here the default is three
(two fused quantise launches and one GEMM with the dequantising epilogue), bit-identical to
the six-launch sequence, which ``fused=False`` still runs through the kernel-level API.
"""
import torch
from ..kernels import gemm_calc_scale, gemm_calc_scale_transpose, gemm_round, gemm_round_transpose, \
    gemm_scale, gemm_scale_x, gemm_scale_y, gemm_int8, gemm_int8_scale, gemm_quantize, gemm_quantize_cols, \
    gemm_quantize_pair, gemm_fp16, gemm_backward_round_scale, gemm_backward_scale_round, transpose, transpose_i8
from ._common import cur_stream


def calc_scale(mat: torch.Tensor, transpose: bool) -> torch.Tensor:
    """reference: torch/gemm.py:5-19"""
    assert mat.is_contiguous() and mat.is_cuda
    b, n, m = mat.size()
    out = torch.empty((b, m if transpose else n), dtype=torch.half, device=mat.device)
    fn = gemm_calc_scale_transpose if transpose else gemm_calc_scale
    fn(b, n, m, mat.data_ptr(), out.data_ptr(), cur_stream())
    return out


def round_i8(mat: torch.Tensor, scale: torch.Tensor, transpose: bool) -> torch.Tensor:
    """reference: torch/gemm.py:21-38"""
    assert mat.is_contiguous() and mat.is_cuda
    assert scale.is_contiguous() and scale.is_cuda
    b, n, m = mat.size()
    out = torch.empty(mat.size(), dtype=torch.int8, device=mat.device)
    fn = gemm_round_transpose if transpose else gemm_round
    fn(b, n, m, mat.data_ptr(), scale.data_ptr(), out.data_ptr(), cur_stream())
    return out


def quantize(mat: torch.Tensor, transpose: bool):
    """calc_scale + round_i8 in one launch; returns (scale, int8 tensor)."""
    assert mat.is_contiguous() and mat.is_cuda and mat.dtype == torch.half
    b, n, m = mat.size()
    scale = torch.empty((b, m if transpose else n), dtype=torch.half, device=mat.device)
    out = torch.empty(mat.size(), dtype=torch.int8, device=mat.device)
    gemm_quantize(b, n, m, mat.data_ptr(), scale.data_ptr(), out.data_ptr(), transpose, cur_stream())
    return scale, out


def quantize_k_major(mat: torch.Tensor, k_is_dim1: bool):
    """Quantise along K and return (scale, int8 tensor with K as the last, contiguous dim):
    for an operand stored (b, rows, K) that is `quantize(mat, False)`; for one stored (b, K, cols)
    the per-column quantisation of `quantize(mat, True)` with the result written transposed,
    (b, cols, K).  Same scales and int8 values either way."""
    if not k_is_dim1:
        return quantize(mat, False)
    assert mat.is_contiguous() and mat.is_cuda and mat.dtype == torch.half
    b, k, cols = mat.size()
    scale = torch.empty((b, cols), dtype=torch.half, device=mat.device)
    out = torch.empty((b, cols, k), dtype=torch.int8, device=mat.device)
    gemm_quantize_cols(b, k, cols, mat.data_ptr(), scale.data_ptr(), out.data_ptr(), True, cur_stream())
    return scale, out


def _dims(quantA, quantB, aT, bT):
    M = quantA.size(2) if aT else quantA.size(1)
    K = quantA.size(1) if aT else quantA.size(2)
    N = quantB.size(1) if bT else quantB.size(2)
    return M, K, N


def gemm_and_scale(quantA, scaleA, quantB, scaleB, aT, bT, fused=True) -> torch.Tensor:
    """reference: torch/gemm.py:40-82.  The operands are swapped in the kernel call exactly as
    there (:45-52) so the (M, N) product comes out row-major.  One of the scales may be None
    (the backward products): the accumulator is then scaled along the other side only."""
    M, K, N = _dims(quantA, quantB, aT, bT)
    batch = max(quantA.size(0), quantB.size(0))
    result_fp = torch.empty((batch, M, N), dtype=torch.float16, device=quantA.device)
    if fused:
        # The MFMA tile kernel reads both operands with K contiguous; an int8 operand given the other
        # way round (the backward products) costs one transposed copy, far less than the general kernel.
        if aT:
            quantA, aT = _transposed_copy_i8(quantA), False
        if not bT:
            quantB, bT = _transposed_copy_i8(quantB), True
        # A missing scale is a vector of ones: (acc * s) * 1 rounds exactly as gemm_scale_x / gemm_scale_y
        # do, and the int32 accumulators never travel through memory.
        if scaleA is None:
            scaleA = torch.ones((1, M), dtype=torch.half, device=quantA.device)
        if scaleB is None:
            scaleB = torch.ones((1, N), dtype=torch.half, device=quantA.device)
        gemm_int8_scale(N, K, M, quantB.size(0), quantA.size(0), bT, aT,
                        quantB.data_ptr(), quantA.data_ptr(),
                        scaleA.data_ptr(), scaleB.data_ptr(),
                        scaleA.size(0) == 1, scaleB.size(0) == 1,
                        result_fp.data_ptr(), cur_stream())
        return result_fp
    result_i32 = torch.empty((batch, M, N), dtype=torch.int32, device=quantA.device)
    gemm_int8(N, K, M, quantB.size(0), quantA.size(0), bT, aT,
              quantB.data_ptr(), quantA.data_ptr(), result_i32.data_ptr(), cur_stream())
    if scaleA is not None and scaleB is not None:
        gemm_scale(batch, M, N, result_i32.data_ptr(), scaleA.data_ptr(), scaleB.data_ptr(),
                   result_fp.data_ptr(), quantA.size(0) == 1, quantB.size(0) == 1, cur_stream())
    elif scaleA is not None:
        gemm_scale_x(batch, M, N, result_i32.data_ptr(), scaleA.data_ptr(), result_fp.data_ptr(), cur_stream())
    else:
        assert scaleB is not None
        gemm_scale_y(batch, M, N, result_i32.data_ptr(), scaleB.data_ptr(), result_fp.data_ptr(), cur_stream())
    return result_fp


class GEMMInt8(torch.autograd.Function):
    @staticmethod
    def forward(ctx, A: torch.Tensor, aT: bool, B: torch.Tensor, bT: bool, fused: bool = True):
        """A: (batchA, M, K) [(batchA, K, M) if aT], B: (batchB, K, N) [(batchB, N, K) if bT]
        -> (batch, M, N) fp16.  reference: torch/gemm.py:84-113"""
        assert A.is_cuda and B.is_cuda and A.device == B.device
        assert A.is_contiguous() and B.is_contiguous()
        assert A.dtype == torch.half and B.dtype == torch.half
        if fused:
            # both operands are brought to K-major int8 while they are quantised, so every
            # layout runs on the fast GEMM kernel: A (bA, M, K) and B (bB, N, K)
            if not aT and bT and A.size(2) == B.size(2):
                # both already K-major: one launch quantises the two of them
                scale_A = torch.empty(A.shape[:2], dtype=torch.half, device=A.device)
                scale_B = torch.empty(B.shape[:2], dtype=torch.half, device=A.device)
                quantized_A = torch.empty(A.shape, dtype=torch.int8, device=A.device)
                quantized_B = torch.empty(B.shape, dtype=torch.int8, device=A.device)
                gemm_quantize_pair(A.size(0) * A.size(1), A.data_ptr(), scale_A.data_ptr(), quantized_A.data_ptr(),
                                   B.size(0) * B.size(1), B.data_ptr(), scale_B.data_ptr(), quantized_B.data_ptr(),
                                   A.size(2), cur_stream())
            else:
                scale_A, quantized_A = quantize_k_major(A, aT)
                scale_B, quantized_B = quantize_k_major(B, not bT)
            # the int8 tensors are held as (bA, M, K) and (bB, N, K) whatever the operand layout was
            ctx.stored = (False, True)
        else:
            scale_A = calc_scale(A, aT)
            scale_B = calc_scale(B, not bT)
            quantized_A = round_i8(A, scale_A, aT)
            quantized_B = round_i8(B, scale_B, not bT)
            ctx.stored = (aT, bT)
        ctx.save_for_backward(scale_A, quantized_A, scale_B, quantized_B)
        ctx.layout = (aT, bT)
        return gemm_and_scale(quantized_A, scale_A, quantized_B, scale_B, ctx.stored[0], ctx.stored[1], fused)

    @staticmethod
    def backward(ctx, grad_f: torch.Tensor):
        """reference: torch/gemm.py:115-186.  grad_A = int8(grad * scale_B, row scales) x quantized_B and
        grad_B = int8(grad * scale_A, column scales)^T x quantized_A, each dequantised by the new
        scales only (the other operand's scales went into the gradient before rounding)."""
        assert grad_f.is_contiguous() and grad_f.is_cuda and grad_f.dtype == torch.float16
        scale_A, quantized_A, scale_B, quantized_B = ctx.saved_tensors
        aT, bT = ctx.stored
        batch, m, n = grad_f.size()
        st = cur_stream()

        scale_G_a = torch.empty((batch, m), dtype=torch.half, device=grad_f.device)
        quant_G_a = torch.empty((batch, m, n), dtype=torch.int8, device=grad_f.device)
        gemm_backward_round_scale(batch, m, n, grad_f.data_ptr(), scale_B.data_ptr(), quant_G_a.data_ptr(),
                                  scale_G_a.data_ptr(), scale_B.size(0) == 1, st)
        if ctx.stored == (False, True):
            # The fused forward holds quantized_A as (bA, M, K) and quantized_B as (bB, N, K).  Each gradient is
            # formed directly in the layout its operand came in, from operands with the contraction index
            # contiguous: no product on the general kernel and no transposition of a result.
            in_aT, in_bT = ctx.layout
            qB_t = _rows_padded_i8(_transposed_copy_i8(quantized_B))    # (bB, K, N)
            quant_G_a = _rows_padded_i8(quant_G_a)                      # both contracted over N
            if in_aT:       # grad_A (b, K, M) = qB_t x quant_G_a^T, scaled per column m
                grad_A = gemm_and_scale(qB_t, None, quant_G_a, scale_G_a, False, True)
            else:           # grad_A (b, M, K) = quant_G_a x qB_t^T, scaled per row m
                grad_A = gemm_and_scale(quant_G_a, scale_G_a, qB_t, None, False, True)
            del scale_G_a, quant_G_a, qB_t
            scale_G_b = torch.empty((batch, n), dtype=torch.half, device=grad_f.device)
            quant_G_b = torch.empty((batch, m, n), dtype=torch.int8, device=grad_f.device)
            gemm_backward_scale_round(batch, m, n, grad_f.data_ptr(), scale_A.data_ptr(), quant_G_b.data_ptr(),
                                      scale_G_b.data_ptr(), scale_A.size(0) == 1, st)
            qG_t = _rows_padded_i8(_transposed_copy_i8(quant_G_b))      # (b, N, M)
            del quant_G_b
            qA_t = _rows_padded_i8(_transposed_copy_i8(quantized_A))    # (bA, K, M); both contracted over M
            if in_bT:       # grad_B (b, N, K) = qG_t x qA_t^T, scaled per row n
                grad_B = gemm_and_scale(qG_t, scale_G_b, qA_t, None, False, True)
            else:           # grad_B (b, K, N) = qA_t x qG_t^T, scaled per column n
                grad_B = gemm_and_scale(qA_t, None, qG_t, scale_G_b, False, True)
            if scale_A.size(0) == 1 and grad_A.size(0) > 1:
                grad_A = grad_A.sum(dim=0, keepdim=True)
            if scale_B.size(0) == 1 and grad_B.size(0) > 1:
                grad_B = grad_B.sum(dim=0, keepdim=True)
            return grad_A, None, grad_B, None, None
        if aT:
            grad_A = gemm_and_scale(quantized_B, None, quant_G_a, scale_G_a, bT, True)
        else:
            grad_A = gemm_and_scale(quant_G_a, scale_G_a, quantized_B, None, False, not bT)
        del scale_G_a, quant_G_a

        scale_G_b = torch.empty((batch, n), dtype=torch.half, device=grad_f.device)
        quant_G_b = torch.empty((batch, m, n), dtype=torch.int8, device=grad_f.device)
        gemm_backward_scale_round(batch, m, n, grad_f.data_ptr(), scale_A.data_ptr(), quant_G_b.data_ptr(),
                                  scale_G_b.data_ptr(), scale_A.size(0) == 1, st)
        if bT:
            grad_B = gemm_and_scale(quant_G_b, scale_G_b, quantized_A, None, True, aT)
        else:
            grad_B = gemm_and_scale(quantized_A, None, quant_G_b, scale_G_b, not aT, False)

        if scale_A.size(0) == 1 and grad_A.size(0) > 1:
            grad_A = grad_A.sum(dim=0, keepdim=True)
        if scale_B.size(0) == 1 and grad_B.size(0) > 1:
            grad_B = grad_B.sum(dim=0, keepdim=True)
        # back to the layout the operands came in
        if ctx.layout[0] != aT:
            grad_A = grad_A.transpose(1, 2).contiguous()
        if ctx.layout[1] != bT:
            grad_B = grad_B.transpose(1, 2).contiguous()
        return grad_A, None, grad_B, None, None


def _transposed_copy_i8(x: torch.Tensor) -> torch.Tensor:
    out = torch.empty((x.size(0), x.size(2), x.size(1)), dtype=torch.int8, device=x.device)
    transpose_i8(x.size(0), x.size(1), x.size(2), x.data_ptr(), out.data_ptr(), cur_stream())
    return out


def _rows_padded_i8(x: torch.Tensor) -> torch.Tensor:
    """A (b, r, k) operand that is contracted over k, with its rows lengthened by zeros to a multiple of 128
    bytes when k is not a multiple of 64: padded on both operands of a product the zeros add nothing, and the
    tile kernel's whole-slab path applies whatever k is (at k = 500 it is several times faster than the kernels
    for ragged rows, and the copy costs two passes over the operand)."""
    k = x.size(2)
    if k % 64 == 0 or k < 128:
        return x
    padded = torch.zeros((x.size(0), x.size(1), (k + 127) // 128 * 128), dtype=torch.int8, device=x.device)
    padded[:, :, :k].copy_(x)
    return padded


def _transposed_copy(x: torch.Tensor) -> torch.Tensor:
    out = torch.empty((x.size(0), x.size(2), x.size(1)), dtype=torch.half, device=x.device)
    transpose(x.size(0), x.size(1), x.size(2), x.data_ptr(), out.data_ptr(), cur_stream())
    return out


def gemm_pth_fp16(A: torch.Tensor, aT: bool, B: torch.Tensor, bT: bool) -> torch.Tensor:
    """reference: torch/gemm.py:189-203; operands are passed swapped to the kernel so that the
    (M, N) result comes out row-major.  The MFMA tile kernel is fastest with K as the contiguous
    dimension of both operands (A as (b, M, K), B as (b, N, K)).  An operand given the other way
    round is read as it lies (2-byte LDS reads build the MFMA fragments, 20-60 % more time in
    the product) unless the product is so large next to the operand that one transposed copy of it
    is cheaper: measured break-even at about 2048 rows of the other operand for B, 512 for A."""
    M, K, N = _dims(A, B, aT, bT)
    if K % 64 == 0 and N % 8 == 0 and M * K < 2 ** 31 and N * K < 2 ** 31:
        if aT and ((N > 512 and K > 128) or M % 8 != 0):     # (short K: the product is bound by writing its output)
            A, aT = _transposed_copy(A), False
        if not bT and M > 2048 and K > 128:
            B, bT = _transposed_copy(B), True
    out = torch.empty((max(A.size(0), B.size(0)), M, N), dtype=torch.half, device=A.device)
    gemm_fp16(N, K, M, B.size(0), A.size(0), bT, aT, B.data_ptr(), A.data_ptr(), out.data_ptr(), cur_stream())
    return out


class GEMMFloat(torch.autograd.Function):
    @staticmethod
    def forward(ctx, A: torch.Tensor, aT: bool, B: torch.Tensor, bT: bool):
        """fp16 product with fp32 accumulation.  reference: torch/gemm.py:205-217 (cuBLASLt there)."""
        assert A.is_cuda and B.is_cuda and A.device == B.device
        assert A.is_contiguous() and B.is_contiguous()
        assert A.dtype == torch.half and B.dtype == torch.half
        ctx.save_for_backward(A, B)
        ctx.aT = aT
        ctx.bT = bT
        return gemm_pth_fp16(A, aT, B, bT)

    @staticmethod
    def backward(ctx, grad_f):
        """reference: torch/gemm.py:219-239"""
        assert grad_f.is_cuda and grad_f.is_contiguous() and grad_f.dtype == torch.float16
        aT, bT = ctx.aT, ctx.bT
        A, B = ctx.saved_tensors
        grad_A = gemm_pth_fp16(B, bT, grad_f, True) if aT else gemm_pth_fp16(grad_f, False, B, not bT)
        grad_B = gemm_pth_fp16(grad_f, True, A, aT) if bT else gemm_pth_fp16(A, not aT, grad_f, False)
        if A.size(0) == 1 and grad_A.size(0) > 1:
            grad_A = grad_A.sum(dim=0, keepdim=True)
        if B.size(0) == 1 and grad_B.size(0) > 1:
            grad_B = grad_B.sum(dim=0, keepdim=True)
        return grad_A, None, grad_B, None


def bmm(A: torch.Tensor, aT: bool, B: torch.Tensor, bT: bool, int8: bool = False, fused: bool = True) -> torch.Tensor:
    assert A.ndim == 3
    assert B.ndim == 3
    if int8:
        return GEMMInt8.apply(A, aT, B, bT, fused)
    return GEMMFloat.apply(A, aT, B, bT)
