"""fp16 transpose of the two inner dimensions, signature of cpm_kernels/kernels/transpose.py."""
from ..library import cpmk
from .base import DevicePointer, CUDAStream, _stream


def transpose(batch: int, n: int, m: int,
              inp: DevicePointer,    # (batch, n, m) fp16
              out: DevicePointer,    # (batch, m, n) fp16
              stream: CUDAStream):
    """reference: kernels/transpose.py:11-29"""
    cpmk.transpose(batch, n, m, inp, out, _stream(stream))


def transpose_i8(batch: int, n: int, m: int,
                 inp: DevicePointer,    # (batch, n, m) int8
                 out: DevicePointer,    # (batch, m, n) int8
                 stream: CUDAStream):
    """The same for int8 tensors (no counterpart in the reference: its cuBLASLt product reads int8
    operands in either layout, kernels/gemm.py:127-186)."""
    cpmk.transpose_i8(batch, n, m, inp, out, _stream(stream))
