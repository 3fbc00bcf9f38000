"""The allocation-free layernorm entry point (cpmk_layernorm_forward_noalloc) against
cpmk_layernorm_forward, through the C-ABI, bit for bit.  It is for callers that cannot allocate;
the reference has no such call."""
import numpy as np
import pytest
import torch

from cpm_kernels_amd.library import cpmk
from util import stream, to_np, assert_bits_equal

pytestmark = pytest.mark.gpu


def _pair(gpu, shape, seed, eps=1e-5, rd_mean=True, inplace=False):
    b, n, m = shape
    print("case no-alloc layernorm", shape, seed, eps, rd_mean, inplace, flush=True)
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(b, n, m, generator=g) * 1.5 + 0.3).half().to(gpu)
    ref = torch.full_like(x, 7.0)
    cpmk.layernorm_forward(b, n, m, x.data_ptr(), ref.data_ptr(), eps, int(rd_mean), stream())
    got = x.clone() if inplace else torch.full_like(x, -7.0)
    src = got if inplace else x
    cpmk.layernorm_forward_noalloc(b, n, m, src.data_ptr(), got.data_ptr(), eps, int(rd_mean), stream())
    assert_bits_equal(to_np(got), to_np(ref), "noalloc %s" % (shape,))
    assert bool(torch.isfinite(got).all())


def test_two_calls_in_a_row_second_smaller(gpu):
    """Config-3 size (256 of the 2048 slots), then a smaller tall input that reuses the first
    slots of the same array, then the first size again."""
    _pair(gpu, (8, 4096, 512), 51)
    _pair(gpu, (2, 1536, 192), 52)
    _pair(gpu, (8, 4096, 512), 53, eps=1e-3, rd_mean=False)
    cpmk.async_status()


@pytest.mark.parametrize("shape", [(3, 2048, 64), (1, 8192, 64 * 32), (2, 1025, 72), (4, 5000, 136)])
def test_team_shapes(gpu, shape):
    _pair(gpu, shape, 60 + shape[1] % 7)
    _pair(gpu, shape, 61 + shape[1] % 7, inplace=True)
    cpmk.async_status()


@pytest.mark.parametrize("shape", [(5, 768, 512), (7, 100, 30), (32, 4096, 1), (2, 16384, 64), (0, 4096, 512)])
def test_shapes_that_need_no_scratch(gpu, shape):
    """Short columns, unaligned shapes, the decode form and columns beyond the team limit run on kernels
    without packet slots: any size is accepted."""
    _pair(gpu, shape, 70)


def test_sizes_beyond_the_scratch_are_refused(gpu):
    x = torch.zeros(17, 4096, 1024, dtype=torch.half, device=gpu)      # 17 * 16 tiles * 8 parts of 512 rows = 2176 slots > 2048
    y = torch.full_like(x, 3.0)
    with pytest.raises(RuntimeError, match="exceeds a size limit"):
        cpmk.layernorm_forward_noalloc(17, 4096, 1024, x.data_ptr(), y.data_ptr(), 1e-5, 1, stream())
    torch.cuda.synchronize()
    assert bool((y == 3.0).all()), "a refused call must not write"
    _pair(gpu, (16, 4096, 1024), 80)                                   # exactly 2048 slots
    _pair(gpu, (1, 16384 - 8192, 2048 * 8), 81)                        # 256 tiles * 8 parts of 1024 rows = 2048 slots


def test_graph_capture_and_replay(gpu):
    """The call can be recorded into a HIP graph (nothing in it allocates, creates an event or clears
    memory from the host) and replayed with changing inputs; eager work runs between the replays."""
    print("case no-alloc layernorm under graph capture", flush=True)
    g = torch.Generator().manual_seed(90)
    x = torch.randn(8, 4096, 512, generator=g).half().to(gpu)
    y = torch.empty_like(x); ref = torch.empty_like(x)
    cpmk.layernorm_forward_noalloc(8, 4096, 512, x.data_ptr(), y.data_ptr(), 1e-5, 1, stream())   # first call on the device outside capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        cpmk.layernorm_forward_noalloc(8, 4096, 512, x.data_ptr(), y.data_ptr(), 1e-5, 1, stream())
    for i in range(4):
        x.copy_((torch.randn(8, 4096, 512, generator=g) * (i + 1)).half())
        y.fill_(0)
        graph.replay()
        torch.cuda.synchronize()
        cpmk.layernorm_forward(8, 4096, 512, x.data_ptr(), ref.data_ptr(), 1e-5, 1, stream())
        assert_bits_equal(to_np(y), to_np(ref), "replay %d" % i)
    cpmk.async_status()
