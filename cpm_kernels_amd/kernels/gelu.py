"""GELU launchers with the signatures of cpm_kernels/kernels/gelu.py."""
from ..library import cpmk
from .base import DevicePointer, CUDAStream, _stream


def gelu_forward(batch: int, n: int,
                 mat: DevicePointer, out: DevicePointer,
                 stream: CUDAStream):
    """reference: kernels/gelu.py:13-30"""
    cpmk.gelu_forward(batch, n, mat, out, _stream(stream))


def gelu_inplace_forward(batch: int, n: int,
                         mat: DevicePointer,
                         stream: CUDAStream):
    """reference: kernels/gelu.py:32-48"""
    cpmk.gelu_forward(batch, n, mat, mat, _stream(stream))


def gelu_backward(batch: int, n: int,
                  grad_out: DevicePointer, mat: DevicePointer, grad: DevicePointer,
                  stream: CUDAStream):
    """grad = gelu'(mat) * grad_out.  reference: kernels/gelu.py:50-69"""
    cpmk.gelu_backward(batch, n, grad_out, mat, grad, _stream(stream))
