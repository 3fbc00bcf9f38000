"""``has_nan_inf`` with the interface of cpm_kernels/torch/utils.py."""
from typing import Optional
import torch
from ..kernels import has_nan_inf as kn_has_nan_inf
from ._common import cur_stream, check_half


def has_nan_inf(x: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Sets ``out`` (a one-element bool tensor) to True when x holds an inf or NaN and leaves it as
    it was otherwise, like the reference (torch/utils.py:5-13); an ``out`` made here starts False
    (the reference hands back uninitialised memory in that case)."""
    check_half(x)
    if out is None:
        out = torch.zeros(1, dtype=torch.bool, device=x.device)[0]
    kn_has_nan_inf(x.numel(), x.data_ptr(), out.data_ptr(), cur_stream())
    return out
