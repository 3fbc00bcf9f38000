"""Plain-torch CPU formulations of the path's operators -- TEST INFRASTRUCTURE ONLY.

Own restatements of the torch formulations the reference's test-suite compares its kernels
with; used as the loose (tolerance) check in tests/ and timed as the CPU baseline by bench.py.
They are whole-op formulations in fp32, not kernel-exact restatements (those are in
cpmk_oracle.c).
"""
import math

import torch


def fake_quant_rows(x: torch.Tensor) -> torch.Tensor:
    """tests/test_gemm.py:8-13 of the reference: fp32 scale = absmax/127 over the last dim,
    round(x/scale)*scale."""
    scale = x.abs().amax(dim=-1, keepdim=True) / 127
    return torch.round(x / scale) * scale


def real_bmm(a: torch.Tensor, aT: bool, b: torch.Tensor, bT: bool, int8: bool) -> torch.Tensor:
    """tests/test_gemm.py:25-41: operands brought to (batch, M, K) and (batch, K, N); with int8
    both are fake-quantised in fp32 over their LAST dim (for the second operand that is N, not
    K -- the reference test does exactly this) and multiplied in fp32."""
    if a.ndim == 2:
        a = a[None]
    if b.ndim == 2:
        b = b[None]
    if aT:
        a = a.transpose(-1, -2)
    if bT:
        b = b.transpose(-1, -2)
    if not int8:
        return torch.matmul(a, b)
    dt = a.dtype
    return torch.matmul(fake_quant_rows(a.float()), fake_quant_rows(b.float())).to(dt)


def quant_bmm_rowwise(a: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """What the kernel path computes for A (b, M, K) and W (b, N, K), in fp32: both operands
    quantised along K, product, no fp16 rounding of scales."""
    return torch.matmul(fake_quant_rows(a.float()), fake_quant_rows(w.float()).transpose(-1, -2))


def layernorm_dim1(x, weight, bias, eps):
    """cpm_kernels/torch/layernorm.py:181-196: fp32, var = E[x^2] - E[x]^2 over dim 1."""
    xf = x.float()
    ex2 = (xf * xf).mean(dim=1, keepdim=True)
    if bias is not None:
        ex = xf.mean(dim=1, keepdim=True)
        xf = (xf - ex) * torch.rsqrt(ex2 - ex * ex + eps)
        xf = xf * weight.float()[None, :, None] + bias.float()[None, :, None]
    else:
        xf = xf * torch.rsqrt(ex2 + eps) * weight.float()[None, :, None]
    return xf.to(x.dtype)


def softmax_dim1(x):
    """cpm_kernels/torch/softmax.py:39-40 (in fp32 on the CPU)."""
    return torch.softmax(x.float(), dim=1).to(x.dtype)


def gelu_tanh(x):
    """cpm_kernels/torch/gelu.py:47-51."""
    xf = x.float()
    return (0.5 * xf * (1.0 + torch.tanh(0.7978845608028654 * xf * (1.0 + 0.044715 * xf * xf)))).to(x.dtype)


def t5_bucket(rel, bidirectional, num_buckets, max_distance):
    """HF-T5 relative_position_bucket as in cpm_kernels/torch/position_embedding.py:84-109;
    rel = key_pos - query_pos."""
    offset = torch.zeros_like(rel)
    if bidirectional:
        num_buckets //= 2
        offset = (rel > 0).long() * num_buckets
        rel = rel.abs()
    else:
        rel = (-rel).clamp(min=0)
    max_exact = num_buckets // 2
    large = max_exact + (torch.log(rel.float() / max_exact) / math.log(max_distance / max_exact)
                         * (num_buckets - max_exact)).long()
    large = large.clamp(max=num_buckets - 1)
    return offset + torch.where(rel < max_exact, rel, large)


def position_bias(weight, query_len, key_len, bidirectional, num_buckets, max_distance):
    """(heads, key_len, query_len) bias, position_embedding.py:111-125."""
    q = torch.arange(query_len)[:, None]
    k = torch.arange(key_len)[None, :]
    buckets = t5_bucket(k - q, bidirectional, num_buckets, max_distance)     # (q, k)
    return weight[:, buckets].permute(0, 2, 1).contiguous()                  # (heads, k, q)
