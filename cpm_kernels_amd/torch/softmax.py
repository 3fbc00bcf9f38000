"""Softmax over dim 1 with the interface of cpm_kernels/torch/softmax.py."""
import torch
from ..kernels import softmax_forward, softmax_backward, softmax_inplace_forward
from ._common import cur_stream, check_half


class OpSoftmax(torch.autograd.Function):
    """reference: torch/softmax.py:4-35"""

    @staticmethod
    def forward(ctx, x: torch.Tensor):
        check_half(x, 3)
        out = torch.empty(x.size(), device=x.device, dtype=torch.half)
        softmax_forward(x.size(0), x.size(1), x.size(2), x.data_ptr(), out.data_ptr(), cur_stream())
        ctx.save_for_backward(out)
        return out

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        check_half(grad_output, 3)
        out = ctx.saved_tensors[0]
        grad = torch.empty(grad_output.size(), device=grad_output.device, dtype=torch.half)
        softmax_backward(grad_output.size(0), grad_output.size(1), grad_output.size(2), out.data_ptr(),
                         grad_output.data_ptr(), grad.data_ptr(), cur_stream())
        return grad


def softmax(x: torch.Tensor) -> torch.Tensor:
    return OpSoftmax.apply(x)


def softmaxTH(x: torch.Tensor) -> torch.Tensor:
    return torch.nn.functional.softmax(x, dim=1)


def softmax_inplace(x: torch.Tensor) -> None:
    check_half(x, 3)
    softmax_inplace_forward(x.size(0), x.size(1), x.size(2), x.data_ptr(), cur_stream())
