"""tanh-GELU with the interface of cpm_kernels/torch/gelu.py."""
import torch
from ..kernels import gelu_forward, gelu_backward, gelu_inplace_forward
from ._common import cur_stream, check_half


class OpGeLU(torch.autograd.Function):
    """reference: torch/gelu.py:4-42"""

    @staticmethod
    def forward(ctx, x: torch.Tensor):
        check_half(x)
        ctx.save_for_backward(x)
        ret = torch.empty_like(x)
        gelu_forward(x.size(0), x.stride(0), x.data_ptr(), ret.data_ptr(), cur_stream())
        return ret

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        x = ctx.saved_tensors[0]
        check_half(grad_output)
        grad = torch.empty_like(grad_output)
        gelu_backward(x.size(0), x.stride(0), grad_output.data_ptr(), x.data_ptr(), grad.data_ptr(), cur_stream())
        return grad


def gelu(x: torch.Tensor) -> torch.Tensor:
    return OpGeLU.apply(x)


def geluTH(x: torch.Tensor) -> torch.Tensor:
    """OpenAI tanh form (torch/gelu.py:47-54)."""
    return 0.5 * x * (1.0 + torch.tanh(0.7978845608028654 * x * (1.0 + 0.044715 * x * x)))


gelu_impl = geluTH      # the reference's name for the same formulation (torch/gelu.py:42-45)


def gelu_inplace(x: torch.Tensor) -> None:
    check_half(x)
    gelu_inplace_forward(x.size(0), x.stride(0), x.data_ptr(), cur_stream())
