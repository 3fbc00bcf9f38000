"""MI355X-native implementation of the int8 quantized-GEMM inference path of cpm_kernels.

``cpm_kernels_amd.kernels`` keeps the call signatures of ``cpm_kernels.kernels``; the CUDA
driver / cuBLASLt ctypes layer underneath is replaced by one C-ABI shared library of
hand-written HIP kernels for gfx950 (include/cpmk.h).  ``cpm_kernels_amd.torch`` (imported
on demand; it needs PyTorch) holds the wrappers of ``cpm_kernels.torch`` for this path.
"""
from . import library
from .kernels import *  # noqa: F401,F403
from .library.cpmk import check  # noqa: F401  (raise a pending asynchronous kernel failure)
