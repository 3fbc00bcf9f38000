"""Relative position bias launchers with the signatures of cpm_kernels/kernels/position_bucket.py."""
from ..library import cpmk
from .base import DevicePointer, CUDAStream, _stream


def position_embedding_init(num_buckets: int, max_distance: int,
                            out: DevicePointer,    # (max_distance)  int32
                            bidirectional: bool,
                            stream: CUDAStream):
    """reference: kernels/position_bucket.py:14-30"""
    cpmk.position_embedding_init(num_buckets, max_distance, out, int(bool(bidirectional)), _stream(stream))


def position_embedding_forward(query_len: int, key_len: int, num_buckets: int, max_distance: int,
                               num_heads: int,
                               position_mapping: DevicePointer,   # (max_distance)  int32
                               weight: DevicePointer,             # (num_heads, num_bucket)  fp16
                               out: DevicePointer,                # (num_heads, key_len, query_len)  fp16
                               bidirectional: bool,
                               stream: CUDAStream):
    """reference: kernels/position_bucket.py:32-58"""
    cpmk.position_embedding_forward(query_len, key_len, num_buckets, max_distance, num_heads, position_mapping,
                                    weight, out, int(bool(bidirectional)), _stream(stream))


def position_embedding_step(query_pos: int, key_len: int, num_buckets: int, max_distance: int,
                            num_heads: int,
                            position_mapping: DevicePointer,   # (max_distance)  int32
                            weight: DevicePointer,             # (num_heads, num_bucket)  fp16
                            out: DevicePointer,                # (num_heads, key_len)  fp16
                            bidirectional: bool,
                            stream: CUDAStream):
    """reference: kernels/position_bucket.py:88-113"""
    cpmk.position_embedding_step(query_pos, key_len, num_buckets, max_distance, num_heads, position_mapping,
                                 weight, out, int(bool(bidirectional)), _stream(stream))


def position_embedding_backward(query_len: int, key_len: int, num_buckets: int, max_distance: int,
                                num_heads: int,
                                position_mapping: DevicePointer,   # (max_distance)  int32
                                grad_out: DevicePointer,           # (num_heads, key_len, query_len)  fp16
                                grad: DevicePointer,               # (num_heads, num_bucket)  fp16
                                bidirectional: bool,
                                stream: CUDAStream):
    """reference: kernels/position_bucket.py:60-86"""
    cpmk.position_embedding_backward(query_len, key_len, num_buckets, max_distance, num_heads, position_mapping,
                                     grad_out, grad, int(bool(bidirectional)), _stream(stream))
