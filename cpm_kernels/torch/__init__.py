"""``cpm_kernels.torch``: same objects as ``cpm_kernels_amd.torch`` (needs PyTorch).

The package namespace carries the public names of the reference's torch/__init__.py:1-14
(where ``gelu``, ``mask``, ``softmax`` and ``transpose`` are functions); every submodule is
registered in ``sys.modules`` as the module object of the implementation, so
``from cpm_kernels.torch.softmax import OpSoftmax`` and ``import cpm_kernels.torch.utils``
resolve exactly as they do against the reference."""
import importlib
import sys

from cpm_kernels_amd.torch import *  # noqa: F401,F403

SUBMODULES = ("arith", "embedding", "gelu", "gemm", "layernorm", "mask", "position_embedding",
              "softmax", "transpose", "utils")

for _name in SUBMODULES:
    _mod = importlib.import_module("cpm_kernels_amd.torch." + _name)
    sys.modules[__name__ + "." + _name] = _mod
    # a function of the same name keeps the attribute (star import above); otherwise the module does
    if _name not in globals():
        globals()[_name] = _mod
