"""Elementwise helpers the path's callers use, with the signatures of cpm_kernels/kernels/arith.py."""
from ..library import cpmk
from .base import DevicePointer, CUDAStream, _stream


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


def arith_global_scale(n: int,
                       inp: DevicePointer,    # (n,) fp16
                       scale: float,
                       out: DevicePointer,    # (n,) fp16
                       stream: CUDAStream):
    """out = fp16(float(x) * scale).  reference: kernels/arith.py:24-41"""
    cpmk.arith_global_scale(n, inp, scale, out, _stream(stream))


def arith_element_mul(batch: int, n: int,
                      x: DevicePointer,      # (batch, n)  fp16
                      y: DevicePointer,      # (batch, n)  fp16
                      out: DevicePointer,    # (batch, n)  fp16
                      stream: CUDAStream):
    """out = x * y.  reference: kernels/arith.py:68-91"""
    assert n % 2 == 0
    cpmk.arith_element_mul(batch, n, x, y, out, _stream(stream))


def arith_batch_add_forward(batch: int, n: int,
                            x: DevicePointer,      # (batch, n)  fp16
                            y: DevicePointer,      # (n)         fp16
                            out: DevicePointer,    # (batch, n)  fp16
                            stream: CUDAStream):
    """out = x + y[None, :].  reference: kernels/arith.py:93-116"""
    assert n % 2 == 0
    cpmk.arith_batch_add_forward(batch, n, x, y, out, _stream(stream))


def arith_batch_add_backward(batch: int, n: int,
                             grad_out: DevicePointer,    # (batch, n)  fp16
                             grad: DevicePointer,        # (n)         fp16
                             stream: CUDAStream):
    """grad = grad_out.sum(0).  reference: kernels/arith.py:118-133"""
    cpmk.arith_batch_add_backward(batch, n, grad_out, grad, _stream(stream))


def arith_ln_add(batch: int, n: int, m: int,
                 inp: DevicePointer,     # (batch, n, m)  fp16
                 beta: DevicePointer,    # (n)            fp16
                 out: DevicePointer,     # (batch, n, m)  fp16
                 stream: CUDAStream):
    """out = x + beta[None, :, None].  reference: kernels/arith.py:163-188"""
    assert m % 2 == 0
    cpmk.arith_ln_add(batch, n, m, inp, beta, out, _stream(stream))


def arith_ln_div(batch: int, n: int, m: int,
                 inp: DevicePointer,      # (batch, n, m)  fp16
                 alpha: DevicePointer,    # (n)            fp16
                 out: DevicePointer,      # (batch, n, m)  fp16
                 stream: CUDAStream):
    """out = x * (1 / alpha)[None, :, None] with the reciprocal rounded to fp16 first.
    reference: kernels/arith.py:216-240"""
    assert m % 2 == 0
    cpmk.arith_ln_div(batch, n, m, inp, alpha, out, _stream(stream))


def arith_ln_sub_div(batch: int, n: int, m: int,
                     inp: DevicePointer,      # (batch, n, m)  fp16
                     alpha: DevicePointer,    # (n)            fp16
                     beta: DevicePointer,     # (n)            fp16
                     out: DevicePointer,      # (batch, n, m)  fp16
                     stream: CUDAStream):
    """out = (x - beta) / alpha evaluated as one fp16 fma with fp16(1/alpha) and fp16(-beta/alpha).
    reference: kernels/arith.py:242-269"""
    assert m % 2 == 0
    cpmk.arith_ln_sub_div(batch, n, m, inp, alpha, beta, out, _stream(stream))


def arith_ln_mul_backward(batch: int, n: int, m: int,
                          inp: DevicePointer,         # (batch, n, m)  fp16
                          grad_out: DevicePointer,    # (batch, n, m)  fp16
                          grad: DevicePointer,        # (n)            fp16
                          stream: CUDAStream):
    """grad = (x * grad_out).sum((0, 2)).  reference: kernels/arith.py:271-289"""
    cpmk.arith_ln_mul_backward(batch, n, m, inp, grad_out, grad, _stream(stream))


def arith_ln_add_backward(batch: int, n: int, m: int,
                          grad_out: DevicePointer,    # (batch, n, m)  fp16
                          grad: DevicePointer,        # (n)            fp16
                          stream: CUDAStream):
    """grad = grad_out.sum((0, 2)).  reference: kernels/arith.py:291-307"""
    cpmk.arith_ln_add_backward(batch, n, m, grad_out, grad, _stream(stream))


def arith_batch_mul_add(batch: int, n: int,
                        x: DevicePointer,        # (batch, n)
                        alpha: DevicePointer,    # (n)
                        beta: DevicePointer,     # (n)
                        out: DevicePointer,      # (batch, n)
                        stream: CUDAStream):
    """out = x * alpha[None, :] + beta[None, :] (fp16 fma).  reference: kernels/arith.py:309-331"""
    assert n % 2 == 0
    cpmk.arith_batch_mul_add(batch, n, x, alpha, beta, out, _stream(stream))


def arith_batch_mul(batch: int, n: int,
                    x: DevicePointer,        # (batch, n)
                    alpha: DevicePointer,    # (n)
                    out: DevicePointer,      # (batch, n)
                    stream: CUDAStream):
    """out = x * alpha[None, :].  reference: kernels/arith.py:333-354"""
    assert n % 2 == 0
    cpmk.arith_batch_mul(batch, n, x, alpha, out, _stream(stream))
