"""Padding mask with the interface of cpm_kernels/torch/mask.py ."""
import torch
from ..kernels import mask as mask_kernel
from ._common import cur_stream, check_half


def _check(x, mask):
    check_half(x, 3)
    assert mask.is_contiguous() and mask.is_cuda and mask.dtype == torch.bool and mask.ndim == 2
    assert x.device == mask.device
    assert mask.size() == (x.size(0), x.size(2))


class OpMask(torch.autograd.Function):
    """reference: torch/mask.py:4-41; the gradient is the incoming gradient with masked positions zeroed."""

    @staticmethod
    def forward(ctx, x: torch.Tensor, mask: torch.Tensor, value: float) -> torch.Tensor:
        _check(x, mask)
        out = torch.empty(x.size(), dtype=torch.float16, device=x.device)
        mask_kernel(x.size(0), x.size(1), x.size(2), x.data_ptr(), mask.data_ptr(), value, out.data_ptr(),
                    cur_stream())
        ctx.save_for_backward(mask)
        return out

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        mask = ctx.saved_tensors[0]
        check_half(grad_output, 3)
        grad = torch.empty(grad_output.size(), dtype=torch.float16, device=grad_output.device)
        mask_kernel(grad_output.size(0), grad_output.size(1), grad_output.size(2), grad_output.data_ptr(), mask.data_ptr(),
                    0.0, grad.data_ptr(), cur_stream())
        return grad, None, None


def mask(x: torch.Tensor, mask: torch.Tensor, value: float) -> torch.Tensor:
    return OpMask.apply(x, mask, value)


def mask_inplace(x: torch.Tensor, mask: torch.Tensor, value: float) -> None:
    _check(x, mask)
    mask_kernel(x.size(0), x.size(1), x.size(2), x.data_ptr(), mask.data_ptr(), value, x.data_ptr(), cur_stream())


def maskTH(x: torch.Tensor, mask: torch.Tensor, value: float) -> torch.Tensor:
    return torch.where(mask[:, None, :], x, torch.scalar_tensor(value, device=x.device, dtype=x.dtype))
