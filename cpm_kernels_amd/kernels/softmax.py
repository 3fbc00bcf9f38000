"""Softmax launchers with the signatures of cpm_kernels/kernels/softmax.py."""
from ..library import cpmk
from .base import DevicePointer, CUDAStream, _stream


def softmax_forward(batch: int, n: int, m: int,
                    inp: DevicePointer,    # (batch, n, m)
                    out: DevicePointer,    # (batch, n, m)
                    stream: CUDAStream):
    """reference: kernels/softmax.py:14-30"""
    cpmk.softmax_forward(batch, n, m, inp, out, _stream(stream))


def softmax_inplace_forward(batch: int, n: int, m: int,
                            inp: DevicePointer,    # (batch, n, m)
                            stream: CUDAStream):
    """reference: kernels/softmax.py:32-46"""
    cpmk.softmax_forward(batch, n, m, inp, inp, _stream(stream))


def softmax_step_inplace(batch: int, n: int,
                         x: DevicePointer,    # (batch, n)
                         stream: CUDAStream):
    """reference: kernels/softmax.py:68-81"""
    cpmk.softmax_step_inplace(batch, n, x, _stream(stream))


def softmax_backward(batch: int, n: int, m: int,
                     out: DevicePointer,         # (batch, n, m)
                     grad_out: DevicePointer,    # (batch, n, m)
                     grad: DevicePointer,        # (batch, n, m)
                     stream: CUDAStream):
    """grad = out * (grad_out - (out * grad_out).sum(1)).  reference: kernels/softmax.py:48-66"""
    cpmk.softmax_backward(batch, n, m, out, grad_out, grad, _stream(stream))
