"""fp16 transpose of the two inner dimensions, signature of cpm_kernels/kernels/transpose.py."""
from ..library import cpmk
from .base import DevicePointer, CUDAStream, _stream


def transpose(batch: int, n: int, m: int,
              inp: DevicePointer,    # (batch, n, m) fp16
              out: DevicePointer,    # (batch, m, n) fp16
              stream: CUDAStream):
    """reference: kernels/transpose.py:11-29"""
    cpmk.transpose(batch, n, m, inp, out, _stream(stream))
