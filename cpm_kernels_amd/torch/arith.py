"""The three elementwise wrappers the inference path uses, with the interface of
cpm_kernels/torch/arith.py (ln_mul_add, ln_mul, element_add; forward only)."""
import torch
from ..kernels import arith_ln_mul_add, arith_ln_mul, arith_element_add
from ._common import cur_stream, check_half, InferenceOnly


def _ln_args(x, alpha, beta=None):
    check_half(x, 3)
    check_half(alpha, 1)
    assert alpha.size(0) == x.size(1)
    if beta is not None:
        check_half(beta, 1)
        assert beta.size(0) == x.size(1)
    return x.size(0), x.size(1), x.size(2)


class OpLnMulAdd(InferenceOnly):
    @staticmethod
    def forward(ctx, x, alpha, beta):
        b, n, m = _ln_args(x, alpha, beta)
        out = torch.empty_like(x)
        arith_ln_mul_add(b, n, m, x.data_ptr(), alpha.data_ptr(), beta.data_ptr(), out.data_ptr(), cur_stream())
        return out


class OpLnMul(InferenceOnly):
    @staticmethod
    def forward(ctx, x, alpha):
        b, n, m = _ln_args(x, alpha)
        out = torch.empty_like(x)
        arith_ln_mul(b, n, m, x.data_ptr(), alpha.data_ptr(), out.data_ptr(), cur_stream())
        return out


class OpElementAdd(InferenceOnly):
    @staticmethod
    def forward(ctx, x, y):
        check_half(x)
        check_half(y)
        assert x.size() == y.size()
        out = torch.empty_like(x)
        arith_element_add(x.size(0), x.stride(0), x.data_ptr(), y.data_ptr(), out.data_ptr(), cur_stream())
        return out


def ln_mul_add(x, alpha, beta):
    return OpLnMulAdd.apply(x, alpha, beta)


def ln_mul_add_inplace(x, alpha, beta) -> None:
    b, n, m = _ln_args(x, alpha, beta)
    arith_ln_mul_add(b, n, m, x.data_ptr(), alpha.data_ptr(), beta.data_ptr(), x.data_ptr(), cur_stream())


def ln_mul_addTH(x, alpha, beta):
    return x * alpha[None, :, None] + beta[None, :, None]


def ln_mul(x, alpha):
    return OpLnMul.apply(x, alpha)


def ln_mul_inplace(x, alpha) -> None:
    b, n, m = _ln_args(x, alpha)
    arith_ln_mul(b, n, m, x.data_ptr(), alpha.data_ptr(), x.data_ptr(), cur_stream())


def ln_mulTH(x, alpha):
    return x * alpha[None, :, None]


def element_add(x, y):
    return OpElementAdd.apply(x, y)


def element_add_inplace(x, y) -> None:
    check_half(x)
    check_half(y)
    assert x.size() == y.size()
    arith_element_add(x.size(0), x.stride(0), x.data_ptr(), y.data_ptr(), x.data_ptr(), cur_stream())


def element_addTH(x, y):
    return x + y
