"""``cpm_kernels.torch``: same objects as ``cpm_kernels_amd.torch`` (needs PyTorch)."""
import sys

import cpm_kernels_amd.torch as _impl
from cpm_kernels_amd.torch import *  # noqa: F401,F403

for _name in ("gemm", "layernorm", "softmax", "gelu", "position_embedding", "mask", "arith"):
    sys.modules[__name__ + "." + _name] = getattr(_impl, _name)
    globals()[_name] = getattr(_impl, _name)
