"""LayerNorm over dim 1 of (batch, hidden, seq) with the interface of
cpm_kernels/torch/layernorm.py."""
import torch
from ..kernels import layernorm_forward, layernorm_inplace_forward, layernorm_affine_forward, \
    layernorm_forward_v, layernorm_forward_mv, layernorm_backward_v, layernorm_backward_mv, \
    arith_ln_mul_add, arith_ln_mul, arith_ln_add_backward, arith_ln_mul_backward
from ._common import cur_stream, check_half


class OpLayerNorm(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x: torch.Tensor, eps: float, weight: torch.Tensor, bias, fused: bool = True):
        """bias given: mean-subtracting norm then y*weight+bias (OpLayerNormMean,
        torch/layernorm.py:7-29); bias None: RMS norm then y*weight (OpLayerNormNoMean, :88-111)."""
        check_half(x, 3)
        check_half(weight, 1)
        b, n, m = x.size()
        out = torch.empty((b, n, m), device=x.device, dtype=torch.float16)
        rd_mean = bias is not None
        ctx.save_for_backward(x, weight)
        ctx.eps = eps
        ctx.rd_mean = rd_mean
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

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        """The reference's sequence (torch/layernorm.py:31-86, 113-156): the normalised tensor and its
        statistics are recomputed, the affine gradients are two channel sums, and the input
        gradient is the norm's backward kernel applied to grad_output * weight."""
        check_half(grad_output, 3)
        x, weight = ctx.saved_tensors
        b, n, m = x.size()
        st = cur_stream()
        half = dict(device=x.device, dtype=torch.float16)
        layer_out = torch.empty((b, n, m), **half)
        var = torch.empty((b, m), **half)
        mean = torch.empty((b, m), **half) if ctx.rd_mean else None
        if ctx.rd_mean:
            layernorm_forward_mv(b, n, m, x.data_ptr(), layer_out.data_ptr(), mean.data_ptr(), var.data_ptr(), ctx.eps, st)
        else:
            layernorm_forward_v(b, n, m, x.data_ptr(), layer_out.data_ptr(), var.data_ptr(), ctx.eps, st)
        grad_bias = None
        if ctx.rd_mean:
            grad_bias = torch.empty((n,), **half)
            arith_ln_add_backward(b, n, m, grad_output.data_ptr(), grad_bias.data_ptr(), st)
        grad_weight = torch.empty((n,), **half)
        arith_ln_mul_backward(b, n, m, layer_out.data_ptr(), grad_output.data_ptr(), grad_weight.data_ptr(), st)
        grad_x = layer_out                     # its contents are no longer needed
        arith_ln_mul(b, n, m, grad_output.data_ptr(), weight.data_ptr(), grad_x.data_ptr(), st)
        grad = torch.empty_like(x)
        if ctx.rd_mean:
            layernorm_backward_mv(b, n, m, x.data_ptr(), grad_x.data_ptr(), mean.data_ptr(), var.data_ptr(), grad.data_ptr(), st)
        else:
            layernorm_backward_v(b, n, m, x.data_ptr(), grad_x.data_ptr(), var.data_ptr(), grad.data_ptr(), st)
        return grad, None, grad_weight, grad_bias, None


class OpLayerNormMean(OpLayerNorm):
    """The reference's name and argument list (x, eps, weight, bias) for the mean-subtracting
    norm (torch/layernorm.py:7-86)."""

    @staticmethod
    def forward(ctx, x: torch.Tensor, eps: float, weight: torch.Tensor, bias: torch.Tensor):
        assert bias is not None
        return OpLayerNorm.forward(ctx, x, eps, weight, bias)

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        return OpLayerNorm.backward(ctx, grad_output)[:4]


class OpLayerNormNoMean(OpLayerNorm):
    """The reference's name and argument list (x, eps, weight) for the RMS norm
    (torch/layernorm.py:88-156)."""

    @staticmethod
    def forward(ctx, x: torch.Tensor, eps: float, weight: torch.Tensor):
        return OpLayerNorm.forward(ctx, x, eps, weight, None)

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        return OpLayerNorm.backward(ctx, grad_output)[:3]


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
