"""Elementwise fp16 wrappers with the interface of cpm_kernels/torch/arith.py: each op as an
autograd function, an in-place variant and a plain-torch ``TH`` formulation."""
import torch
from ..kernels import arith
from ._common import cur_stream, check_half


def _ln_args(x, alpha=None, beta=None):
    check_half(x, 3)
    for p in (alpha, beta):
        if p is not None:
            check_half(p, 1)
            assert p.device == x.device and p.size(0) == x.size(1)
    return x.size(0), x.size(1), x.size(2)


def _same(x, y):
    check_half(x)
    check_half(y)
    assert x.device == y.device and x.size() == y.size()


def _batched(x, y):
    check_half(x)
    check_half(y)
    assert x.device == y.device and x.size()[1:] == y.size()


# ---- out = x * scale ---------------------------------------------------------------------------
class OpGlobalScale(torch.autograd.Function):
    """reference: torch/arith.py:4-29"""

    @staticmethod
    def forward(ctx, x: torch.Tensor, scale: float):
        check_half(x)
        out = torch.empty(x.size(), device=x.device, dtype=torch.half)
        arith.arith_global_scale(x.numel(), x.data_ptr(), scale, out.data_ptr(), cur_stream())
        ctx.scale = scale
        return out

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        check_half(grad_output)
        grad = torch.empty(grad_output.size(), device=grad_output.device, dtype=torch.half)
        arith.arith_global_scale(grad_output.numel(), grad_output.data_ptr(), ctx.scale, grad.data_ptr(), cur_stream())
        return grad, None


def global_scale(x: torch.Tensor, scale: float) -> torch.Tensor:
    return OpGlobalScale.apply(x, scale)


def global_scaleTH(x: torch.Tensor, scale: float) -> torch.Tensor:
    return x * scale


def global_scale_inplace(x: torch.Tensor, scale: float) -> None:
    check_half(x)
    arith.arith_global_scale(x.numel(), x.data_ptr(), scale, x.data_ptr(), cur_stream())


# ---- out = x + y -------------------------------------------------------------------------------
class OpElementAdd(torch.autograd.Function):
    """reference: torch/arith.py:55-75"""

    @staticmethod
    def forward(ctx, x, y):
        _same(x, y)
        out = torch.empty_like(x)
        arith.arith_element_add(x.size(0), x.stride(0), x.data_ptr(), y.data_ptr(), out.data_ptr(), cur_stream())
        return out

    @staticmethod
    def backward(ctx, grad_output):
        return grad_output, grad_output


def element_add(x, y):
    return OpElementAdd.apply(x, y)


def element_add_inplace(x, y) -> None:
    _same(x, y)
    arith.arith_element_add(x.size(0), x.stride(0), x.data_ptr(), y.data_ptr(), x.data_ptr(), cur_stream())


def element_addTH(x, y):
    return x + y


# ---- out = x * y -------------------------------------------------------------------------------
class OpElementMul(torch.autograd.Function):
    """reference: torch/arith.py:106-146"""

    @staticmethod
    def forward(ctx, x, y):
        _same(x, y)
        out = torch.empty_like(x)
        arith.arith_element_mul(x.size(0), x.stride(0), x.data_ptr(), y.data_ptr(), out.data_ptr(), cur_stream())
        ctx.save_for_backward(x, y)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        check_half(grad_output)
        x, y = ctx.saved_tensors
        grad_x = torch.empty_like(x)
        grad_y = torch.empty_like(y)
        arith.arith_element_mul(x.size(0), x.stride(0), grad_output.data_ptr(), y.data_ptr(), grad_x.data_ptr(), cur_stream())
        arith.arith_element_mul(y.size(0), y.stride(0), x.data_ptr(), grad_output.data_ptr(), grad_y.data_ptr(), cur_stream())
        return grad_x, grad_y


def element_mul(x, y):
    return OpElementMul.apply(x, y)


def element_mul_inplace(x, y) -> None:
    _same(x, y)
    arith.arith_element_mul(x.size(0), x.stride(0), x.data_ptr(), y.data_ptr(), x.data_ptr(), cur_stream())


def element_mulTH(x, y):
    return x * y


# ---- out = x + y[None, :] ----------------------------------------------------------------------
class OpBatchedAdd(torch.autograd.Function):
    """reference: torch/arith.py:177-207"""

    @staticmethod
    def forward(ctx, x, y):
        _batched(x, y)
        out = torch.empty_like(x)
        arith.arith_batch_add_forward(x.size(0), x.stride(0), x.data_ptr(), y.data_ptr(), out.data_ptr(), cur_stream())
        return out

    @staticmethod
    def backward(ctx, grad_output):
        check_half(grad_output)
        grad_y = torch.empty(grad_output.size()[1:], device=grad_output.device, dtype=grad_output.dtype)
        arith.arith_batch_add_backward(grad_output.size(0), grad_output.stride(0), grad_output.data_ptr(), grad_y.data_ptr(),
                                       cur_stream())
        return grad_output, grad_y


def batched_add(x, y):
    return OpBatchedAdd.apply(x, y)


def batched_add_inplace(x, y) -> None:
    _batched(x, y)
    arith.arith_batch_add_forward(x.size(0), x.stride(0), x.data_ptr(), y.data_ptr(), x.data_ptr(), cur_stream())


def batched_addTH(x, y):
    return x + y[None, :]


# ---- out = x * alpha[None, :, None] + beta[None, :, None] --------------------------------------
def _ln_param_grads(x, grad_output, want_alpha: bool, want_beta: bool):
    b, n, m = grad_output.size()
    grad_alpha = grad_beta = None
    if want_alpha:
        grad_alpha = torch.empty((n,), device=x.device, dtype=torch.half)
        arith.arith_ln_mul_backward(b, n, m, x.data_ptr(), grad_output.data_ptr(), grad_alpha.data_ptr(), cur_stream())
    if want_beta:
        grad_beta = torch.empty((n,), device=grad_output.device, dtype=torch.half)
        arith.arith_ln_add_backward(b, n, m, grad_output.data_ptr(), grad_beta.data_ptr(), cur_stream())
    return grad_alpha, grad_beta


class OpLnMulAdd(torch.autograd.Function):
    """reference: torch/arith.py:240-292"""

    @staticmethod
    def forward(ctx, x, alpha, beta):
        b, n, m = _ln_args(x, alpha, beta)
        out = torch.empty_like(x)
        arith.arith_ln_mul_add(b, n, m, x.data_ptr(), alpha.data_ptr(), beta.data_ptr(), out.data_ptr(), cur_stream())
        ctx.save_for_backward(x, alpha)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        check_half(grad_output, 3)
        b, n, m = grad_output.size()
        x, alpha = ctx.saved_tensors
        grad_x = torch.empty_like(x)
        arith.arith_ln_mul(b, n, m, grad_output.data_ptr(), alpha.data_ptr(), grad_x.data_ptr(), cur_stream())
        grad_alpha, grad_beta = _ln_param_grads(x, grad_output, True, True)
        return grad_x, grad_alpha, grad_beta


def ln_mul_add(x, alpha, beta):
    return OpLnMulAdd.apply(x, alpha, beta)


def ln_mul_add_inplace(x, alpha, beta) -> None:
    b, n, m = _ln_args(x, alpha, beta)
    arith.arith_ln_mul_add(b, n, m, x.data_ptr(), alpha.data_ptr(), beta.data_ptr(), x.data_ptr(), cur_stream())


def ln_mul_addTH(x, alpha, beta):
    return x * alpha[None, :, None] + beta[None, :, None]


# ---- out = x * alpha[None, :, None] ------------------------------------------------------------
class OpLnMul(torch.autograd.Function):
    """reference: torch/arith.py:328-371"""

    @staticmethod
    def forward(ctx, x, alpha):
        b, n, m = _ln_args(x, alpha)
        out = torch.empty_like(x)
        arith.arith_ln_mul(b, n, m, x.data_ptr(), alpha.data_ptr(), out.data_ptr(), cur_stream())
        ctx.save_for_backward(x, alpha)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        check_half(grad_output, 3)
        b, n, m = grad_output.size()
        x, alpha = ctx.saved_tensors
        grad_x = torch.empty_like(x)
        arith.arith_ln_mul(b, n, m, grad_output.data_ptr(), alpha.data_ptr(), grad_x.data_ptr(), cur_stream())
        grad_alpha, _ = _ln_param_grads(x, grad_output, True, False)
        return grad_x, grad_alpha


def ln_mul(x, alpha):
    return OpLnMul.apply(x, alpha)


def ln_mul_inplace(x, alpha) -> None:
    b, n, m = _ln_args(x, alpha)
    arith.arith_ln_mul(b, n, m, x.data_ptr(), alpha.data_ptr(), x.data_ptr(), cur_stream())


def ln_mulTH(x, alpha):
    return x * alpha[None, :, None]


# ---- out = x + beta[None, :, None] -------------------------------------------------------------
class OpLnAdd(torch.autograd.Function):
    """reference: torch/arith.py:405-438"""

    @staticmethod
    def forward(ctx, x, beta):
        b, n, m = _ln_args(x, None, beta)
        out = torch.empty_like(x)
        arith.arith_ln_add(b, n, m, x.data_ptr(), beta.data_ptr(), out.data_ptr(), cur_stream())
        return out

    @staticmethod
    def backward(ctx, grad_output):
        check_half(grad_output, 3)
        _, grad_beta = _ln_param_grads(grad_output, grad_output, False, True)
        return grad_output, grad_beta


def ln_add(x, beta):
    return OpLnAdd.apply(x, beta)


def ln_add_inplace(x, beta) -> None:
    b, n, m = _ln_args(x, None, beta)
    arith.arith_ln_add(b, n, m, x.data_ptr(), beta.data_ptr(), x.data_ptr(), cur_stream())


def ln_addTH(x, beta):
    return x + beta[None, :, None]


# ---- out = (x - beta[None, :, None]) / alpha[None, :, None]   (no gradient in the reference either) ----
def ln_sub_div(x, alpha, beta):
    """reference: torch/arith.py:471-492"""
    b, n, m = _ln_args(x, alpha, beta)
    out = torch.empty_like(x)
    arith.arith_ln_sub_div(b, n, m, x.data_ptr(), alpha.data_ptr(), beta.data_ptr(), out.data_ptr(), cur_stream())
    return out


def ln_sub_div_inplace(x, alpha, beta) -> None:
    b, n, m = _ln_args(x, alpha, beta)
    arith.arith_ln_sub_div(b, n, m, x.data_ptr(), alpha.data_ptr(), beta.data_ptr(), x.data_ptr(), cur_stream())


def ln_sub_divTH(x, alpha, beta):
    return (x - beta[None, :, None]) / alpha[None, :, None]


# ---- out = x / alpha[None, :, None] ------------------------------------------------------------
def ln_div(x, alpha):
    """reference: torch/arith.py:523-542"""
    b, n, m = _ln_args(x, alpha)
    out = torch.empty_like(x)
    arith.arith_ln_div(b, n, m, x.data_ptr(), alpha.data_ptr(), out.data_ptr(), cur_stream())
    return out


def ln_div_inplace(x, alpha) -> None:
    b, n, m = _ln_args(x, alpha)
    arith.arith_ln_div(b, n, m, x.data_ptr(), alpha.data_ptr(), x.data_ptr(), cur_stream())


def ln_divTH(x, alpha):
    return x / alpha[None, :, None]
