"""Token-embedding gathers with the signatures of cpm_kernels/kernels/embedding.py (forward and
decode step; the backward stages are outside the inference path)."""
from ..library import cpmk
from .base import DevicePointer, CUDAStream, _stream, not_on_path


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


_e = "token embedding backward, kernels/embedding.py"
embedding_backward_stage1 = not_on_path("embedding_backward_stage1", _e)
embedding_backward_stage2 = not_on_path("embedding_backward_stage2", _e)
