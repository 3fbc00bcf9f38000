"""Normalisation launchers with the signatures of cpm_kernels/kernels/layernorm.py."""
from ..library import cpmk
from .base import DevicePointer, CUDAStream, _stream


def layernorm_forward(batch: int, n: int, m: int,
                      mat: DevicePointer,    # (batch, n, m)
                      out: DevicePointer,    # (batch, n, m)
                      eps: float, rd_mean: bool,
                      stream: CUDAStream):
    """reference: kernels/layernorm.py:18-38"""
    cpmk.layernorm_forward(batch, n, m, mat, out, eps, int(bool(rd_mean)), _stream(stream))


def layernorm_inplace_forward(batch: int, n: int, m: int,
                              mat: DevicePointer,    # (batch, n, m)
                              eps: float, rd_mean: bool,
                              stream: CUDAStream):
    """reference: kernels/layernorm.py:40-58"""
    cpmk.layernorm_forward(batch, n, m, mat, mat, eps, int(bool(rd_mean)), _stream(stream))


def layernorm_affine_forward(batch: int, n: int, m: int,
                             mat: DevicePointer,      # (batch, n, m)
                             alpha: DevicePointer,    # (n)
                             beta,                    # (n) or None / 0
                             out: DevicePointer,      # (batch, n, m)
                             eps: float, rd_mean: bool,
                             stream: CUDAStream):
    """layernorm_forward + arith_ln_mul_add / arith_ln_mul in one launch, bit-identical to the
    two-launch sequence of torch/layernorm.py:9-29,88-111."""
    cpmk.layernorm_affine_forward(batch, n, m, mat, alpha, beta or None, out, eps, int(bool(rd_mean)),
                                  _stream(stream))


def layernorm_step(batch: int, n: int,
                   mat: DevicePointer,    # (batch, n)  fp16
                   out: DevicePointer,    # (batch, n)  fp16
                   eps: float, rd_mean: bool,
                   stream: CUDAStream):
    """reference: kernels/layernorm.py:152-171"""
    cpmk.layernorm_step(batch, n, mat, out, eps, int(bool(rd_mean)), _stream(stream))


def layernorm_step_inplace(batch: int, n: int,
                           mat: DevicePointer,    # (batch, n)  fp16
                           eps: float, rd_mean: bool,
                           stream: CUDAStream):
    """reference: kernels/layernorm.py:173-190"""
    cpmk.layernorm_step(batch, n, mat, mat, eps, int(bool(rd_mean)), _stream(stream))


def layernorm_forward_v(batch: int, n: int, m: int,
                        mat: DevicePointer,        # (batch, n, m)
                        out: DevicePointer,        # (batch, n, m)
                        out_var: DevicePointer,    # (batch, m)
                        eps: float,
                        stream: CUDAStream):
    """RMS norm over dim 1 that keeps rsqrt(mean(x^2) + eps) for the backward pass.
    reference: kernels/layernorm.py:60-80"""
    cpmk.layernorm_forward_v(batch, n, m, mat, out, out_var, eps, _stream(stream))


def layernorm_forward_mv(batch: int, n: int, m: int,
                         mat: DevicePointer,         # (batch, n, m)
                         out: DevicePointer,         # (batch, n, m)
                         out_mean: DevicePointer,    # (batch, m)
                         out_var: DevicePointer,     # (batch, m)
                         eps: float,
                         stream: CUDAStream):
    """reference: kernels/layernorm.py:82-104"""
    cpmk.layernorm_forward_mv(batch, n, m, mat, out, out_mean, out_var, eps, _stream(stream))


def layernorm_backward_v(batch: int, n: int, m: int,
                         mat: DevicePointer,         # (batch, n, m)
                         grad_out: DevicePointer,    # (batch, n, m)
                         var: DevicePointer,         # (batch, m)
                         grad: DevicePointer,        # (batch, n, m)
                         stream: CUDAStream):
    """reference: kernels/layernorm.py:106-126"""
    cpmk.layernorm_backward_v(batch, n, m, mat, grad_out, var, grad, _stream(stream))


def layernorm_backward_mv(batch: int, n: int, m: int,
                          mat: DevicePointer,         # (batch, n, m)
                          grad_out: DevicePointer,    # (batch, n, m)
                          mean: DevicePointer,        # (batch, m)
                          var: DevicePointer,         # (batch, m)
                          grad: DevicePointer,        # (batch, n, m)
                          stream: CUDAStream):
    """reference: kernels/layernorm.py:128-150"""
    cpmk.layernorm_backward_mv(batch, n, m, mat, grad_out, mean, var, grad, _stream(stream))
