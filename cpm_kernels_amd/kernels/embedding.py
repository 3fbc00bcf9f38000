"""Token-embedding gathers with the signatures of cpm_kernels/kernels/embedding.py ."""
from ..library import cpmk
from .base import DevicePointer, CUDAStream, _stream


def embedding_forward(batch: int,
                      hidden_size: int,          # hidden size
                      seq_len: int,              # sequence length
                      ids: DevicePointer,        # (batch, seq_len) int32
                      weights: DevicePointer,    # (vocab_size, hidden_size) fp16
                      out: DevicePointer,        # (batch, hidden_size, seq_len) fp16
                      stream: CUDAStream):
    """reference: kernels/embedding.py:14-34"""
    cpmk.embedding_forward(batch, hidden_size, seq_len, ids, weights, out, _stream(stream))


def embedding_step(batch: int, embedding_size: int,
                   ids: DevicePointer,            # (batch,) int32
                   weights: DevicePointer,        # (vocab_size, embedding_size) fp16
                   out: DevicePointer,            # (batch, embedding_size) fp16
                   stream: CUDAStream):
    """reference: kernels/embedding.py:88-105"""
    cpmk.embedding_step(batch, embedding_size, ids, weights, out, _stream(stream))


def embedding_backward_stage1(batch: int, seq_len: int, hidden_size: int,
                              grad_out: DevicePointer,        # (batch * n, m)
                              argsort_ids: DevicePointer,     # (batch, n)
                              sorted_ids: DevicePointer,      # (batch, n)
                              grad: DevicePointer,            # (vocab_size, m)
                              aux_grad: DevicePointer,        # (batch, m)
                              aux_grad_idx: DevicePointer,    # (batch)
                              stream: CUDAStream):
    """Sums runs of equal sorted ids inside each batch entry.  reference: kernels/embedding.py:36-65"""
    cpmk.embedding_backward_stage1(batch, seq_len, hidden_size, grad_out, argsort_ids, sorted_ids, grad, aux_grad,
                                   aux_grad_idx, _stream(stream))


def embedding_backward_stage2(batch: int, hidden_size: int,
                              aux_grad: DevicePointer,        # (batch, m)
                              aux_grad_idx: DevicePointer,    # (batch)
                              grad: DevicePointer,            # (vocab_size, m)
                              stream: CUDAStream):
    """Adds the per-entry tail runs into grad.  reference: kernels/embedding.py:67-86"""
    cpmk.embedding_backward_stage2(batch, hidden_size, aux_grad, aux_grad_idx, grad, _stream(stream))
