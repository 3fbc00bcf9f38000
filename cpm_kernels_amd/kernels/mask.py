"""Padding mask launcher with the signature of cpm_kernels/kernels/mask.py."""
from ..library import cpmk
from .base import DevicePointer, CUDAStream, _stream


def mask(batch: int, n: int, m: int,
         inp: DevicePointer,     # (batch, n, m)  fp16
         mask: DevicePointer,    # (batch, m)     int8 / bool
         value: float,
         out: DevicePointer,     # (batch, n, m)  fp16
         stream: CUDAStream):
    """out[b,i,j] = mask[b,j] ? inp[b,i,j] : value.  reference: kernels/mask.py:12-35"""
    cpmk.mask(batch, n, m, inp, mask, value, out, _stream(stream))
