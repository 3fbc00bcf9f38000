"""fp16 transpose of the two inner dims with the interface of cpm_kernels/torch/transpose.py."""
import torch
from ..kernels import transpose as transpose_kernel
from ._common import cur_stream, check_half


def _run(x: torch.Tensor) -> torch.Tensor:
    check_half(x, 3)
    out = torch.empty((x.size(0), x.size(2), x.size(1)), dtype=torch.half, device=x.device)
    transpose_kernel(x.size(0), x.size(1), x.size(2), x.data_ptr(), out.data_ptr(), cur_stream())
    return out


class OpTranspose(torch.autograd.Function):
    """reference: torch/transpose.py:5-28"""

    @staticmethod
    def forward(ctx, x: torch.Tensor):
        return _run(x)

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        return _run(grad_output)


def transpose(x: torch.Tensor) -> torch.Tensor:
    return OpTranspose.apply(x)


def transposeTH(x: torch.Tensor) -> torch.Tensor:
    assert x.ndim == 3
    return x.transpose(1, 2)
