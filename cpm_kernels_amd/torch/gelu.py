"""tanh-GELU with the interface of cpm_kernels/torch/gelu.py (forward only)."""
import torch
from ..kernels import gelu_forward, gelu_inplace_forward
from ._common import cur_stream, check_half, InferenceOnly


class OpGeLU(InferenceOnly):
    @staticmethod
    def forward(ctx, x: torch.Tensor):
        check_half(x)
        ret = torch.empty_like(x)
        gelu_forward(x.size(0), x.stride(0), x.data_ptr(), ret.data_ptr(), cur_stream())
        return ret


def gelu(x: torch.Tensor) -> torch.Tensor:
    return OpGeLU.apply(x)


def geluTH(x: torch.Tensor) -> torch.Tensor:
    """OpenAI tanh form (torch/gelu.py:47-54)."""
    return 0.5 * x * (1.0 + torch.tanh(0.7978845608028654 * x * (1.0 + 0.044715 * x * x)))


def gelu_inplace(x: torch.Tensor) -> None:
    check_half(x)
    gelu_inplace_forward(x.size(0), x.stride(0), x.data_ptr(), cur_stream())
