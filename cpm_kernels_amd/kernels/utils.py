"""``cpm_kernels.kernels.utils`` of the reference: helpers of the decode loop."""
from ..library import cpmk
from .base import DevicePointer, CUDAStream, _stream


def copy_data_to_kv(batch: int, buffer_len: int, n: int,
                    inp: DevicePointer,        # (batch, n) fp16
                    out: DevicePointer,        # (batch, buffer_len, n) fp16
                    pos: int,
                    stream: CUDAStream):
    """reference: kernels/utils.py:18-37"""
    assert n % 2 == 0
    cpmk.copy_data_to_kv(batch, buffer_len, n, inp, out, pos, _stream(stream))


def array_add(array: DevicePointer, pos: int, val: int, stream: CUDAStream):
    """array[pos] += val on an int32 device array.  reference: kernels/utils.py:39-53"""
    cpmk.array_add(array, pos, val, _stream(stream))


def adjustify_logits(batch: int, n: int,
                     logits: DevicePointer,       # (batch, n) fp16, updated in place
                     temperature: float, frequency_penalty: float, presence_penalty: float,
                     frequency: DevicePointer,    # (batch, n) int32
                     stream: CUDAStream):
    """reference: kernels/utils.py:55-77"""
    cpmk.adjustify_logits(batch, n, logits, temperature, frequency_penalty, presence_penalty, frequency, _stream(stream))


def copy_extend_buffer(batch: int, old_size: int, nw_size: int,
                       old_buffer: DevicePointer,    # (batch, old_size) fp16
                       new_buffer: DevicePointer,    # (batch, nw_size) fp16
                       stream: CUDAStream):
    """reference: kernels/utils.py:79-96"""
    cpmk.copy_extend_buffer(batch, old_size, nw_size, old_buffer, new_buffer, _stream(stream))


def has_nan_inf(n: int,
                inp: DevicePointer,    # (n,)  fp16
                out: DevicePointer,    # (1,)  bool, set to 1 when an inf/NaN is present, untouched otherwise
                stream: CUDAStream):
    """reference: kernels/utils.py:98-112"""
    cpmk.has_nan_inf(n, inp, out, _stream(stream))


def copy_pos_hidden(batch: int, hidden_size: int, seq_len: int, pos: int,
                    inp: DevicePointer,    # (batch, hidden_size, seq_len) fp16
                    out: DevicePointer,    # (batch, hidden_size) fp16
                    stream: CUDAStream):
    """reference: kernels/utils.py:114-134"""
    cpmk.copy_pos_hidden(batch, hidden_size, seq_len, pos, inp, out, _stream(stream))
