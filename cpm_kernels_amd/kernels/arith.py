"""Elementwise helpers the path's callers use, with the signatures of cpm_kernels/kernels/arith.py."""
from ..library import cpmk
from .base import DevicePointer, CUDAStream, _stream, not_on_path


def arith_element_add(batch: int, n: int,
                      x: DevicePointer,      # (batch, n)  fp16
                      y: DevicePointer,      # (batch, n)  fp16
                      out: DevicePointer,    # (batch, n)  fp16
                      stream: CUDAStream):
    """out = x + y.  reference: kernels/arith.py:43-66"""
    assert n % 2 == 0
    cpmk.arith_element_add(batch, n, x, y, out, _stream(stream))


def arith_ln_mul_add(batch: int, n: int, m: int,
                     inp: DevicePointer,      # (batch, n, m)  fp16
                     alpha: DevicePointer,    # (n)            fp16
                     beta: DevicePointer,     # (n)            fp16
                     out: DevicePointer,      # (batch, n, m)  fp16
                     stream: CUDAStream):
    """out = x * alpha[None, :, None] + beta[None, :, None] (fp16 fma).
    reference: kernels/arith.py:135-161"""
    assert m % 2 == 0
    cpmk.arith_ln_mul_add(batch, n, m, inp, alpha, beta, out, _stream(stream))


def arith_ln_mul(batch: int, n: int, m: int,
                 inp: DevicePointer,      # (batch, n, m)  fp16
                 alpha: DevicePointer,    # (n)            fp16
                 out: DevicePointer,      # (batch, n, m)  fp16
                 stream: CUDAStream):
    """out = x * alpha[None, :, None].  reference: kernels/arith.py:190-214"""
    assert m % 2 == 0
    cpmk.arith_ln_mul(batch, n, m, inp, alpha, out, _stream(stream))


_w = "not used by the inference path, kernels/arith.py"
arith_global_scale = not_on_path("arith_global_scale", _w)
arith_element_mul = not_on_path("arith_element_mul", _w)
arith_batch_add_forward = not_on_path("arith_batch_add_forward", _w)
arith_batch_add_backward = not_on_path("arith_batch_add_backward", _w)
arith_ln_add = not_on_path("arith_ln_add", _w)
arith_ln_sub_div = not_on_path("arith_ln_sub_div", _w)
arith_ln_div = not_on_path("arith_ln_div", _w)
arith_ln_add_backward = not_on_path("arith_ln_add_backward", _w)
arith_ln_mul_backward = not_on_path("arith_ln_mul_backward", _w)
arith_batch_mul_add = not_on_path("arith_batch_mul_add", _w)
arith_batch_mul = not_on_path("arith_batch_mul", _w)
