"""Quantisation, int8 GEMM and dequantisation launchers with the signatures of
cpm_kernels/kernels/gemm.py.  Arithmetic contracts are stated in include/cpmk.h."""
from ..library import cpmk
from .base import DevicePointer, CUDAStream, _stream


def gemm_round(batch: int, n: int, m: int,
               mat: DevicePointer,      # (b, n, m)  fp16
               scale: DevicePointer,    # (b, n)     fp16
               out: DevicePointer,      # (b, n, m)  int8
               stream: CUDAStream):
    """reference: kernels/gemm.py:21-41"""
    cpmk.gemm_round(batch, n, m, mat, scale, out, _stream(stream))


def gemm_round_transpose(batch: int, n: int, m: int,
                         mat: DevicePointer,    # (b, n, m)  fp16
                         scale: DevicePointer,  # (b, m)     fp16
                         out: DevicePointer,    # (b, n, m)  int8
                         stream: CUDAStream):
    """reference: kernels/gemm.py:43-63"""
    cpmk.gemm_round_transpose(batch, n, m, mat, scale, out, _stream(stream))


def gemm_scale(batch: int, n: int, m: int,
               mat: DevicePointer,        # (b, n, m)  int32
               scale_x: DevicePointer,    # (b, n)     fp16
               scale_y: DevicePointer,    # (b, m)     fp16
               out: DevicePointer,        # (b, n, m)  fp16
               broad_cast_x: bool, broad_cast_y: bool,
               stream: CUDAStream):
    """reference: kernels/gemm.py:65-89"""
    cpmk.gemm_scale(batch, n, m, mat, scale_x, scale_y, out, int(bool(broad_cast_x)),
                    int(bool(broad_cast_y)), _stream(stream))


def gemm_calc_scale(batch: int, n: int, m: int,
                    mat: DevicePointer,    # (b, n, m) fp16
                    out: DevicePointer,    # (b, n)    fp16
                    stream: CUDAStream):
    """reference: kernels/gemm.py:91-107"""
    cpmk.gemm_calc_scale(batch, n, m, mat, out, _stream(stream))


def gemm_calc_scale_transpose(batch: int, n: int, m: int,
                              inp: DevicePointer,    # (b, n, m) fp16
                              out: DevicePointer,    # (b, m)    fp16
                              stream: CUDAStream):
    """reference: kernels/gemm.py:109-125"""
    cpmk.gemm_calc_scale_transpose(batch, n, m, inp, out, _stream(stream))


def gemm_int8(m: int, k: int, n: int,
              batchA: int, batchB: int,
              aT: bool, bT: bool,
              A: DevicePointer,      # (bA, k, m) int8   [(bA, m, k) if aT]
              B: DevicePointer,      # (bB, n, k) int8   [(bB, k, n) if bT]
              out: DevicePointer,    # (max(bA, bB), n, m) int32
              stream: CUDAStream):
    """reference: kernels/gemm.py:127-186 (cuBLASLt); same asserts (:139-140)."""
    assert m % 4 == 0 and n % 4 == 0 and k % 4 == 0
    assert batchA == batchB or batchA == 1 or batchB == 1
    cpmk.gemm_int8(m, k, n, batchA, batchB, int(bool(aT)), int(bool(bT)), A, B, out, _stream(stream))


def gemm_int8_scale(m: int, k: int, n: int,
                    batchA: int, batchB: int,
                    aT: bool, bT: bool,
                    A: DevicePointer, B: DevicePointer,
                    scale_row: DevicePointer,   # fp16 per output row j:  (n) or (batch, n)
                    scale_col: DevicePointer,   # fp16 per output col i:  (m) or (batch, m)
                    broad_cast_row: bool, broad_cast_col: bool,
                    out: DevicePointer,         # (max(bA, bB), n, m) fp16
                    stream: CUDAStream):
    """gemm_int8 with the gemm_scale epilogue fused (no counterpart launcher in the reference;
    it fuses kernels/gemm.py:127-186 and :65-89 as torch/gemm.py:40-64 chains them)."""
    assert m % 4 == 0 and n % 4 == 0 and k % 4 == 0
    assert batchA == batchB or batchA == 1 or batchB == 1
    cpmk.gemm_int8_scale(m, k, n, batchA, batchB, int(bool(aT)), int(bool(bT)), A, B, scale_row, scale_col,
                         int(bool(broad_cast_row)), int(bool(broad_cast_col)), out, _stream(stream))


def gemm_quantize(batch: int, n: int, m: int,
                  mat: DevicePointer,      # (b, n, m) fp16
                  scale: DevicePointer,    # (b, n) or, transposed, (b, m) fp16
                  out: DevicePointer,      # (b, n, m) int8
                  transpose: bool,
                  stream: CUDAStream):
    """gemm_calc_scale[_transpose] + gemm_round[_transpose] in one call (fuses
    torch/gemm.py:5-38)."""
    cpmk.gemm_quantize(batch, n, m, mat, scale, out, int(bool(transpose)), _stream(stream))


def gemm_quantize_pair(rows0: int, mat0: DevicePointer, scale0: DevicePointer, out0: DevicePointer,
                       rows1: int, mat1: DevicePointer, scale1: DevicePointer, out1: DevicePointer,
                       m: int, stream: CUDAStream):
    """gemm_quantize(transpose=False) of two tensors with rows of length m (rows0 x m fp16 at
    mat0, rows1 x m at mat1) in one launch."""
    cpmk.gemm_quantize_pair(rows0, mat0, scale0, out0, rows1, mat1, scale1, out1, m, _stream(stream))


def gemm_quantize_cols(batch: int, n: int, m: int,
                       mat: DevicePointer,      # (b, n, m) fp16
                       scale: DevicePointer,    # (b, m) fp16
                       out: DevicePointer,      # (b, n, m) int8, or (b, m, n) if out_transposed
                       out_transposed: bool,
                       stream: CUDAStream):
    """gemm_calc_scale_transpose + gemm_round_transpose in one pass (fuses torch/gemm.py:5-38 for
    an operand quantised along dim 1), optionally writing the int8 tensor transposed so that it
    is K-major for gemm_int8."""
    cpmk.gemm_quantize_cols(batch, n, m, mat, scale, out, int(bool(out_transposed)), _stream(stream))


def gemm_scale_x(batch: int, n: int, m: int,
                 mat: DevicePointer,        # (b, n, m)  int32
                 scale_x: DevicePointer,    # (b, n)     fp16
                 out: DevicePointer,        # (b, n, m)  fp16
                 stream: CUDAStream):
    """reference: kernels/gemm.py:309-327"""
    cpmk.gemm_scale_x(batch, n, m, mat, scale_x, out, _stream(stream))


def gemm_scale_y(batch: int, n: int, m: int,
                 mat: DevicePointer,        # (b, n, m)  int32
                 scale_y: DevicePointer,    # (b, m)     fp16
                 out: DevicePointer,        # (b, n, m)  fp16
                 stream: CUDAStream):
    """reference: kernels/gemm.py:329-347"""
    cpmk.gemm_scale_y(batch, n, m, mat, scale_y, out, _stream(stream))


def gemm_fp16(m: int, k: int, n: int,
              batchA: int, batchB: int,
              aT: bool, bT: bool,
              A: DevicePointer,      # (bA, k, m) fp16   [(bA, m, k) if aT]
              B: DevicePointer,      # (bB, n, k) fp16   [(bB, k, n) if bT]
              out: DevicePointer,    # (max(bA, bB), n, m) fp16
              stream: CUDAStream):
    """reference: kernels/gemm.py:188-256 (cuBLASLt); same asserts (:200-201).  fp32 accumulation."""
    assert m % 2 == 0 and n % 2 == 0 and k % 2 == 0
    assert batchA == batchB or batchA == 1 or batchB == 1
    cpmk.gemm_fp16(m, k, n, batchA, batchB, int(bool(aT)), int(bool(bT)), A, B, out, _stream(stream))


def gemm_backward_round_scale(batch: int, n: int, m: int,
                              mat: DevicePointer,        # (batch, n, m) fp16
                              scale_y: DevicePointer,    # (batch, m)    fp16
                              out: DevicePointer,        # (batch, n, m) int8
                              scale_x: DevicePointer,    # (batch, n)    fp16
                              broad_cast_y: bool,
                              stream: CUDAStream):
    """Row scales and int8 rounding of mat * scale_y.  reference: kernels/gemm.py:261-283"""
    cpmk.gemm_backward_round_scale(batch, n, m, mat, scale_y, out, scale_x, int(bool(broad_cast_y)), _stream(stream))


def gemm_backward_scale_round(batch: int, n: int, m: int,
                              mat: DevicePointer,        # (batch, n, m) fp16
                              scale_x: DevicePointer,    # (batch, n)    fp16
                              out: DevicePointer,        # (batch, n, m) int8
                              scale_y: DevicePointer,    # (batch, m)    fp16
                              broad_cast_x: bool,
                              stream: CUDAStream):
    """Column scales and int8 rounding of mat * scale_x.  reference: kernels/gemm.py:285-307"""
    cpmk.gemm_backward_scale_round(batch, n, m, mat, scale_x, out, scale_y, int(bool(broad_cast_x)), _stream(stream))
