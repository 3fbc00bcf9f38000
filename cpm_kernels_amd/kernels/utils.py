"""``cpm_kernels.kernels.utils`` of the reference: decode-loop utilities.  ``copy_data_to_kv`` feeds
the key/value buffers next to the int8 path and is implemented; the others are not on the path,
their names resolve and calls raise NotImplementedError."""
from ..library import cpmk
from .base import DevicePointer, CUDAStream, _stream
from .offpath import has_nan_inf, array_add, adjustify_logits, copy_extend_buffer, copy_pos_hidden  # noqa: F401


def copy_data_to_kv(batch: int, buffer_len: int, n: int,
                    inp: DevicePointer,        # (batch, n) fp16
                    out: DevicePointer,        # (batch, buffer_len, n) fp16
                    pos: int,
                    stream: CUDAStream):
    """reference: kernels/utils.py:18-37"""
    assert n % 2 == 0
    cpmk.copy_data_to_kv(batch, buffer_len, n, inp, out, pos, _stream(stream))
