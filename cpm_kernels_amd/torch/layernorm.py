"""LayerNorm over dim 1 of (batch, hidden, seq) with the interface of
cpm_kernels/torch/layernorm.py (forward only)."""
import torch
from ..kernels import layernorm_forward, layernorm_inplace_forward, layernorm_affine_forward, \
    arith_ln_mul_add, arith_ln_mul
from ._common import cur_stream, check_half, InferenceOnly


class OpLayerNorm(InferenceOnly):
    @staticmethod
    def forward(ctx, x: torch.Tensor, eps: float, weight: torch.Tensor, bias, fused: bool = True):
        """bias given: mean-subtracting norm then y*weight+bias (OpLayerNormMean,
        torch/layernorm.py:7-29); bias None: RMS norm then y*weight (OpLayerNormNoMean, :88-111)."""
        check_half(x, 3)
        check_half(weight, 1)
        b, n, m = x.size()
        out = torch.empty((b, n, m), device=x.device, dtype=torch.float16)
        rd_mean = bias is not None
        if fused:
            layernorm_affine_forward(b, n, m, x.data_ptr(), weight.data_ptr(),
                                     bias.data_ptr() if rd_mean else None, out.data_ptr(), eps, rd_mean,
                                     cur_stream())
            return out
        layernorm_forward(b, n, m, x.data_ptr(), out.data_ptr(), eps, rd_mean, cur_stream())
        if rd_mean:
            arith_ln_mul_add(b, n, m, out.data_ptr(), weight.data_ptr(), bias.data_ptr(), out.data_ptr(), cur_stream())
        else:
            arith_ln_mul(b, n, m, out.data_ptr(), weight.data_ptr(), out.data_ptr(), cur_stream())
        return out


class LayerNorm(torch.nn.Module):
    """reference: torch/layernorm.py:158-172"""

    def __init__(self, hidden_size: int, eps: float = 1e-5, bias=True, fused: bool = True):
        super().__init__()
        self.eps = eps
        self.fused = fused
        self.weight = torch.nn.Parameter(torch.ones(hidden_size))
        self.bias = torch.nn.Parameter(torch.zeros(hidden_size)) if bias else None

    def forward(self, x: torch.Tensor):
        check_half(x, 3)
        assert x.size(1) == self.weight.size(0)
        return OpLayerNorm.apply(x, self.eps, self.weight, self.bias, self.fused)


class LayerNormTH(torch.nn.Module):
    """Plain-torch formulation of the same layer (torch/layernorm.py:174-196):
    fp32, var = E[x^2] - E[x]^2 over dim 1."""

    def __init__(self, hidden_size: int, eps: float = 1e-5, bias=True):
        super().__init__()
        self.eps = eps
        self.weight = torch.nn.Parameter(torch.ones(hidden_size))
        self.bias = torch.nn.Parameter(torch.zeros(hidden_size)) if bias else None

    def forward(self, x: torch.Tensor):
        y = normalizeTH(x.float(), self.eps, self.bias is not None)
        y = y * self.weight[None, :, None]
        if self.bias is not None:
            y = y + self.bias[None, :, None]
        return y.to(x.dtype)


def normalize_inplace(x: torch.Tensor, eps: float, rd_mean: bool):
    """reference: torch/layernorm.py:198-206"""
    check_half(x, 3)
    layernorm_inplace_forward(x.size(0), x.size(1), x.size(2), x.data_ptr(), eps, rd_mean, cur_stream())


def normalizeTH(x: torch.Tensor, eps: float, rd_mean: bool) -> torch.Tensor:
    """reference: torch/layernorm.py:208-218"""
    xf = x.float()
    ex2 = (xf * xf).mean(dim=1, keepdim=True)
    if rd_mean:
        ex = xf.mean(dim=1, keepdim=True)
        xf = (xf - ex) * torch.rsqrt(ex2 - ex * ex + eps)
    else:
        xf = xf * torch.rsqrt(ex2 + eps)
    return xf.to(x.dtype)
