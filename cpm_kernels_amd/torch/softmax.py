"""Softmax over dim 1 with the interface of cpm_kernels/torch/softmax.py (forward only)."""
import torch
from ..kernels import softmax_forward, softmax_inplace_forward
from ._common import cur_stream, check_half, InferenceOnly


class OpSoftmax(InferenceOnly):
    @staticmethod
    def forward(ctx, x: torch.Tensor):
        check_half(x, 3)
        out = torch.empty(x.size(), device=x.device, dtype=torch.half)
        softmax_forward(x.size(0), x.size(1), x.size(2), x.data_ptr(), out.data_ptr(), cur_stream())
        return out


def softmax(x: torch.Tensor) -> torch.Tensor:
    return OpSoftmax.apply(x)


def softmaxTH(x: torch.Tensor) -> torch.Tensor:
    return torch.nn.functional.softmax(x, dim=1)


def softmax_inplace(x: torch.Tensor) -> None:
    check_half(x, 3)
    softmax_inplace_forward(x.size(0), x.size(1), x.size(2), x.data_ptr(), cur_stream())
