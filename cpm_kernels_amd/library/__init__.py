"""Bindings below the kernels layer.  The reference binds libcuda, libcudart, libcublasLt and
libnvrtc here (cpm_kernels/library/__init__.py:1-4); this build needs exactly one library,
the C-ABI ``libcpmk_hip.so`` declared in include/cpmk.h."""
from . import cpmk
