"""T5-style relative position bias with the interface of
cpm_kernels/torch/position_embedding.py ."""
import math
import torch
import torch.nn.functional as F
from ..kernels import position_embedding_init, position_embedding_forward, position_embedding_backward
from ._common import cur_stream, check_half


class OpPositionEmbedding(torch.autograd.Function):
    """reference: torch/position_embedding.py:6-55"""

    @staticmethod
    def forward(ctx, query_len, key_len, num_buckets, max_distance, num_heads, weight: torch.Tensor,
                bidirectional: bool):
        check_half(weight)
        device = weight.device
        mapping = torch.empty((max_distance,), dtype=torch.int32, device=device)
        position_embedding_init(num_buckets, max_distance, mapping.data_ptr(), bidirectional, cur_stream())
        out = torch.empty((num_heads, key_len, query_len), device=device, dtype=torch.float16)
        position_embedding_forward(query_len, key_len, num_buckets, max_distance, num_heads, mapping.data_ptr(),
                                   weight.data_ptr(), out.data_ptr(), bidirectional, cur_stream())
        ctx.save_for_backward(mapping)
        ctx.input_args = (query_len, key_len, num_buckets, max_distance, num_heads, bidirectional)
        return out

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        check_half(grad_output)
        query_len, key_len, num_buckets, max_distance, num_heads, bidirectional = ctx.input_args
        mapping = ctx.saved_tensors[0]
        grad = torch.empty((num_heads, num_buckets), device=grad_output.device, dtype=torch.float16)
        position_embedding_backward(query_len, key_len, num_buckets, max_distance, num_heads, mapping.data_ptr(),
                                    grad_output.data_ptr(), grad.data_ptr(), bidirectional, cur_stream())
        return None, None, None, None, None, grad, None


class PositionEmbedding(torch.nn.Module):
    """reference: torch/position_embedding.py:57-69"""

    def __init__(self, num_heads, num_buckets, max_distance, bidirectional=True):
        super().__init__()
        self.weight = torch.nn.Parameter(torch.randn(num_heads, num_buckets))
        self.num_heads = num_heads
        self.num_buckets = num_buckets
        self.max_distance = max_distance
        self.bidirectional = bidirectional

    def forward(self, key_len, query_len):
        return OpPositionEmbedding.apply(query_len, key_len, self.num_buckets, self.max_distance, self.num_heads,
                                         self.weight, self.bidirectional)


class PositionEmbeddingTH(torch.nn.Module):
    """Plain-torch T5 bucket formulation (torch/position_embedding.py:73-128)."""

    def __init__(self, num_heads, num_buckets, max_distance, bidirectional=True) -> None:
        super().__init__()
        self.num_buckets = num_buckets
        self.num_heads = num_heads
        self.max_distance = max_distance
        self.bidirectional = bidirectional
        self.weight = torch.nn.Parameter(torch.randn(num_heads, num_buckets))

    def relative_position_bucket(self, rel, bidirectional=True, num_buckets=32, max_distance=128):
        offset = 0
        if bidirectional:
            num_buckets //= 2
            offset = (rel > 0).to(torch.long) * num_buckets
            rel = rel.abs()
        else:
            rel = (-rel).clamp(min=0)
        max_exact = num_buckets // 2
        large = max_exact + (torch.log(rel.float() / max_exact) / math.log(max_distance / max_exact)
                             * (num_buckets - max_exact)).to(torch.long)
        large = large.clamp(max=num_buckets - 1)
        return offset + torch.where(rel < max_exact, rel, large)

    def compute_bias(self, query_length, key_length):
        device = self.weight.device
        q = torch.arange(query_length, dtype=torch.long, device=device)[:, None]
        k = torch.arange(key_length, dtype=torch.long, device=device)[None, :]
        buckets = self.relative_position_bucket(k - q, self.bidirectional, self.num_buckets, self.max_distance)
        values = F.embedding(buckets, self.weight.transpose(0, 1))    # (q, k, heads)
        return values.permute([2, 1, 0])                              # (heads, k, q)

    def forward(self, key_length, query_length):
        return self.compute_bias(query_length, key_length)
