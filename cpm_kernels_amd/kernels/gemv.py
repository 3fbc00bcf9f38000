"""Decode GEMV launchers with the signatures of cpm_kernels/kernels/gemv.py."""
from ..library import cpmk
from .base import DevicePointer, CUDAStream, _stream, not_on_path


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


_w = "fp16 GEMV, kernels/gemv.py:82-283"
gemv_fp16 = not_on_path("gemv_fp16", _w)
gemv_fp16_light = not_on_path("gemv_fp16_light", _w)
gemv_fp16_transpose = not_on_path("gemv_fp16_transpose", _w)
gemv_fp16_transpose_light = not_on_path("gemv_fp16_transpose_light", _w)
gemv_broadcast_mat_fp16 = not_on_path("gemv_broadcast_mat_fp16", _w)
gemv_broadcast_mat_fp16_light = not_on_path("gemv_broadcast_mat_fp16_light", _w)
