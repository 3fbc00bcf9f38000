"""What happens when stream capture has used up the packet slots set aside for recorded launches.
A launch recorded into a HIP graph keeps its slots for good (the graph may be replayed at any time),
so the reserve only shrinks; once it is empty the library records kernels that need no packets
instead.  This file is collected late on purpose: after it, every recorded team launch of the process
takes that path."""
import numpy as np
import pytest
import torch

import oracle
import cpm_kernels_amd.kernels as ck
from cpm_kernels_amd.library import cpmk
from util import stream, to_np, assert_bits_equal, assert_close_fp16

pytestmark = pytest.mark.gpu


def test_recorded_launches_beyond_the_reserve_run_without_packets(gpu):
    print("case capture reserve exhausted", flush=True)
    g = torch.Generator().manual_seed(46)
    x = torch.randn(8, 4096, 512, generator=g).half().to(gpu)
    ref = torch.empty_like(x)
    ck.layernorm_forward(8, 4096, 512, x.data_ptr(), ref.data_ptr(), 1e-5, True, stream())
    xt = (torch.randn(2, 4096, 128, generator=g) * 3).half().to(gpu)
    ref_sm = torch.empty_like(xt); ref_sc = torch.empty((2, 128), dtype=torch.half, device=gpu); ref_q = torch.empty((2, 128, 4096), dtype=torch.int8, device=gpu)
    ck.softmax_forward(2, 4096, 128, xt.data_ptr(), ref_sm.data_ptr(), stream())
    ck.gemm_quantize_cols(2, 4096, 128, xt.data_ptr(), ref_sc.data_ptr(), ref_q.data_ptr(), True, stream())
    # a softmax over many column tiles (640: more than two per compute unit), whose tile counters come out of the pool too
    xm = (torch.randn(40, 1024, 1024, generator=g) * 3).half().to(gpu)
    ref_many = torch.empty_like(xm); many = torch.zeros_like(xm)
    ck.softmax_forward(40, 1024, 1024, xm.data_ptr(), ref_many.data_ptr(), stream())
    torch.cuda.synchronize()
    assert cpmk.exchange_capture_slots_left() <= 140 * 256
    ys = [torch.zeros_like(x) for _ in range(4)]
    sm_team = torch.zeros_like(xt); sm = torch.zeros_like(xt); sc = torch.zeros_like(ref_sc); q = torch.zeros_like(ref_q)

    def record(fn):
        g_ = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g_):
            fn()
        return g_

    # The launches recorded on one stream during one capture share a range of slots (they run one after the other):
    # three tall layernorms in one graph take the 256 slots of one ...
    left = cpmk.exchange_capture_slots_left()
    chain = record(lambda: [ck.layernorm_forward(8, 4096, 512, x.data_ptr(), ys[i].data_ptr(), 1e-5, True, stream()) for i in range(3)])
    assert cpmk.exchange_capture_slots_left() == left - 256
    # ... and every capture takes a range of its own: record one launch per graph until the reserve is used up
    graphs = []
    while cpmk.exchange_capture_slots_left() >= 256:           # a tall layernorm of this size takes 256 slots
        graphs.append(record(lambda: ck.layernorm_forward(8, 4096, 512, x.data_ptr(), ys[len(graphs) % 3].data_ptr(), 1e-5, True, stream())))
    sm_graphs = []
    while cpmk.exchange_capture_slots_left() >= 64:            # slots are given out in multiples of 64
        sm_graphs.append(record(lambda: ck.softmax_forward(2, 4096, 128, xt.data_ptr(), sm_team.data_ptr(), stream())))
    assert cpmk.exchange_capture_slots_left() < 64 and len(graphs) >= 3

    def without_packets():
        ck.layernorm_forward(8, 4096, 512, x.data_ptr(), ys[3].data_ptr(), 1e-5, True, stream())
        ck.softmax_forward(2, 4096, 128, xt.data_ptr(), sm.data_ptr(), stream())
        ck.gemm_quantize_cols(2, 4096, 128, xt.data_ptr(), sc.data_ptr(), q.data_ptr(), True, stream())
        ck.softmax_forward(40, 1024, 1024, xm.data_ptr(), many.data_ptr(), stream())
    last = record(without_packets)                             # the reserve is empty: recorded as kernels that need no packets
    for rep in range(2):
        for y in ys:
            y.fill_(0)
        torch.cuda.synchronize()
        chain.replay()
        for g_ in graphs[:4] + graphs[-2:] + sm_graphs:
            g_.replay()
        last.replay()
        torch.cuda.synchronize()
        cpmk.async_status()
        for y in ys[:3]:
            assert_bits_equal(to_np(y), to_np(ref), "replay %d: launches with slots" % rep)
        if sm_graphs:
            assert_bits_equal(to_np(sm_team), to_np(ref_sm), "replay %d: softmax with slots" % rep)
        # without packets the sums are added in another order: the 1e-3 bar of the path's fp16 outputs, against the oracle
        exp = oracle.layernorm_forward(to_np(x), 1e-5, True)
        assert_close_fp16(to_np(ys[3]), exp.astype(np.float64), rtol=1e-3, atol=2e-4, what="replay %d: launches without slots" % rep)
        assert_close_fp16(to_np(sm), to_np(ref_sm).astype(np.float64), rtol=1e-3, atol=1e-6, what="softmax without slots")
        assert_bits_equal(to_np(sc), to_np(ref_sc), "column scales without slots")
        assert_bits_equal(to_np(q), to_np(ref_q), "column int8 without slots")
        # (one tile per workgroup instead of tiles from a counter: the same arithmetic on every column)
        assert_bits_equal(to_np(many), to_np(ref_many), "many-tile softmax without counters")
    # eager launches are not affected
    y = torch.zeros_like(x)
    ck.layernorm_forward(8, 4096, 512, x.data_ptr(), y.data_ptr(), 1e-5, True, stream())
    assert_bits_equal(to_np(y), to_np(ref), "eager launch afterwards")
