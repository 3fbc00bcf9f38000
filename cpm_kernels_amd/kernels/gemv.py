"""Decode GEMV launchers with the signatures of cpm_kernels/kernels/gemv.py."""
from ..library import cpmk
from .base import DevicePointer, CUDAStream, _stream


def gemv_calc_scale(batch: int, n: int,
                    vec: DevicePointer,     # (batch, n)  fp16
                    out: DevicePointer,     # (batch,)    fp16
                    stream: CUDAStream):
    """reference: kernels/gemv.py:18-33"""
    cpmk.gemv_calc_scale(batch, n, vec, out, _stream(stream))


def gemv_round(batch: int, n: int,
               vec: DevicePointer,      # (batch, n)  fp16
               scale: DevicePointer,    # (batch)     fp16
               out: DevicePointer,      # (batch, n)  int8
               stream: CUDAStream):
    """reference: kernels/gemv.py:35-53"""
    cpmk.gemv_round(batch, n, vec, scale, out, _stream(stream))


def gemv_broadcast_mat_int8(batch: int, dim_out: int, dim_in: int,
                            scale_mat: DevicePointer,   # (dim_out,)        fp16
                            mat: DevicePointer,         # (dim_out, dim_in) int8
                            scale_vec: DevicePointer,   # (batch,)          fp16
                            vec: DevicePointer,         # (batch, dim_in)   int8
                            out: DevicePointer,         # (batch, dim_out)  fp16
                            stream: CUDAStream):
    """reference: kernels/gemv.py:56-79"""
    assert dim_in % 4 == 0
    cpmk.gemv_broadcast_mat_int8(batch, dim_out, dim_in, scale_mat, mat, scale_vec, vec, out, _stream(stream))


def gemv_fp16(batch: int, dim_out: int, dim_in: int,
              mat: DevicePointer,     # (batch, dim_out, dim_in) fp16
              vec: DevicePointer,     # (batch, dim_in)   fp16
              out: DevicePointer,     # (batch, dim_out)  fp16
              stream: CUDAStream):
    """reference: kernels/gemv.py:82-127 (cuBLASLt)"""
    cpmk.gemv_fp16(batch, dim_out, dim_in, mat, vec, out, _stream(stream))


def gemv_fp16_light(batch: int, dim_out: int, dim_in: int, mat: DevicePointer, vec: DevicePointer,
                    out: DevicePointer, stream: CUDAStream):
    """reference: kernels/gemv.py:129-149 (the reference's own kernel instead of cuBLASLt)"""
    assert dim_in % 2 == 0
    cpmk.gemv_fp16(batch, dim_out, dim_in, mat, vec, out, _stream(stream))


def gemv_fp16_transpose(batch: int, dim_out: int, dim_in: int,
                        mat: DevicePointer,     # (batch, dim_in, dim_out) fp16
                        vec: DevicePointer,     # (batch, dim_in)   fp16
                        out: DevicePointer,     # (batch, dim_out)  fp16
                        stream: CUDAStream):
    """reference: kernels/gemv.py:151-196 (cuBLASLt)"""
    cpmk.gemv_fp16_transpose(batch, dim_out, dim_in, mat, vec, out, _stream(stream))


def gemv_fp16_transpose_light(batch: int, dim_out: int, dim_in: int, mat: DevicePointer, vec: DevicePointer,
                              out: DevicePointer, stream: CUDAStream):
    """reference: kernels/gemv.py:198-216"""
    cpmk.gemv_fp16_transpose(batch, dim_out, dim_in, mat, vec, out, _stream(stream))


def gemv_broadcast_mat_fp16(batch: int, dim_out: int, dim_in: int,
                            mat: DevicePointer,     # (dim_out, dim_in) fp16
                            vec: DevicePointer,     # (batch, dim_in)   fp16
                            out: DevicePointer,     # (batch, dim_out)  fp16
                            stream: CUDAStream):
    """reference: kernels/gemv.py:218-262 (cuBLASLt)"""
    cpmk.gemv_broadcast_mat_fp16(batch, dim_out, dim_in, mat, vec, out, _stream(stream))


def gemv_broadcast_mat_fp16_light(batch: int, dim_out: int, dim_in: int, mat: DevicePointer, vec: DevicePointer,
                                  out: DevicePointer, stream: CUDAStream):
    """reference: kernels/gemv.py:264-283"""
    assert dim_in % 2 == 0
    cpmk.gemv_broadcast_mat_fp16(batch, dim_out, dim_in, mat, vec, out, _stream(stream))
