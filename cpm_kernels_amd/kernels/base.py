"""Common names of the kernels layer (cpm_kernels/kernels/base.py:7-13 of the reference).

The reference's ``Kernel`` / ``KernelFunction`` classes load a fatbin per .cu file and
launch by name with a grid computed in Python (base.py:15-77).  Here every kernel is a C-ABI
launcher of libcpmk_hip.so, so the wrappers only validate and forward their arguments.
"""
import ctypes

DevicePointer = int
CUDAStream = ctypes.c_void_p     # name kept; on ROCm torch's ``.cuda_stream`` is a hipStream_t


def round_up(x: int, m: int) -> int:
    return (x + m - 1) // m * m


def _stream(stream):
    """Accept an int, None or a ctypes.c_void_p like the reference's launch path does."""
    if isinstance(stream, ctypes.c_void_p):
        return stream
    return ctypes.c_void_p(stream)
