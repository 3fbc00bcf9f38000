import torch


def cur_stream() -> int:
    """Raw hipStream_t of torch's current stream (ROCm builds keep the ``cuda`` names)."""
    return torch.cuda.current_stream().cuda_stream


def check_half(x: torch.Tensor, ndim=None):
    assert x.is_cuda and x.is_contiguous() and x.dtype == torch.float16
    if ndim is not None:
        assert x.ndim == ndim
