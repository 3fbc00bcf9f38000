"""GELU launchers with the signatures of cpm_kernels/kernels/gelu.py."""
from ..library import cpmk
from .base import DevicePointer, CUDAStream, _stream, not_on_path


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


gelu_backward = not_on_path("gelu_backward", "training, kernels/gelu.py:50-69")
