"""Two properties beside parity.  Repeatability: results must not depend on timing (last test).
Pointers that are only 4-byte aligned: torch hands out 256-byte aligned tensors, but a caller's
view into a larger buffer need not be, and the reference asks for nothing beyond the alignment of
its half2 / char4 accesses.  Every 16-byte fast path must step aside for such pointers: each
function is run on aligned tensors and again with every operand moved 4 bytes off, and the two
results must agree (to the bit for the exact kernels).  The dim-1 and elementwise kernels are also run
on buffers that start on an odd element (2 bytes off), which they take as well."""
import sys

import numpy as np
import pytest
import torch

import cpm_kernels_amd.kernels as ck
from util import stream, to_np, assert_bits_equal, assert_close_fp16

pytestmark = pytest.mark.gpu


def _name(*a):
    print("case", *a, flush=True)


SHIFT_BYTES = 4


def shifted(t):
    """The same values at an address SHIFT_BYTES (4 unless a test says otherwise) past a 256-byte boundary."""
    e = max(1, SHIFT_BYTES // t.element_size())
    buf = torch.empty(t.numel() + 64, dtype=t.dtype, device=t.device)
    v = buf[e:e + t.numel()].view(t.shape)
    v.copy_(t)
    assert v.data_ptr() % 16 == e * t.element_size()
    return v


def both(fn, inputs, out_shape, out_dtype, gpu, exact=True, what=""):
    """fn(*pointers of inputs, pointer of out) on aligned and on shifted operands."""
    out_a = torch.zeros(out_shape, dtype=out_dtype, device=gpu)
    fn(*[t.data_ptr() for t in inputs], out_a.data_ptr())
    sh = [shifted(t) for t in inputs]
    out_s = shifted(torch.zeros(out_shape, dtype=out_dtype, device=gpu))
    fn(*[t.data_ptr() for t in sh], out_s.data_ptr())
    if exact:
        assert_bits_equal(to_np(out_s), to_np(out_a), what + ": shifted == aligned")
    else:
        assert_close_fp16(to_np(out_s), to_np(out_a).astype(np.float64), rtol=1e-3, atol=2e-4, what=what + ": shifted vs aligned")
    return out_a


def test_quantised_gemm_path_unaligned(gpu):
    _name("quantise / gemm / dequant, 4-byte aligned pointers")
    g = torch.Generator().manual_seed(31)
    n, k, m = 136, 256, 264
    X = torch.randn(1, n, k, generator=g).half().to(gpu)
    W = (torch.randn(1, m, k, generator=g) * 0.05).half().to(gpu)
    s = stream()
    sx = both(lambda x, o: ck.gemm_calc_scale(1, n, k, x, o, s), [X], (1, n), torch.half, gpu, what="calc_scale")
    sw = both(lambda x, o: ck.gemm_calc_scale(1, m, k, x, o, s), [W], (1, m), torch.half, gpu, what="calc_scale W")
    qx = both(lambda x, sc, o: ck.gemm_round(1, n, k, x, sc, o, s), [X, sx], (1, n, k), torch.int8, gpu, what="round")
    qw = both(lambda x, sc, o: ck.gemm_round(1, m, k, x, sc, o, s), [W, sw], (1, m, k), torch.int8, gpu, what="round W")
    both(lambda x, o: ck.gemm_calc_scale_transpose(1, n, k, x, o, s), [X], (1, k), torch.half, gpu, what="calc_scale_transpose")
    for aT, bT, A, B in ((True, False, qw, qx), (False, False, qw.transpose(1, 2).contiguous(), qx),
                         (True, True, qw, qx.transpose(1, 2).contiguous())):
        acc = both(lambda a, b, o: ck.gemm_int8(m, k, n, 1, 1, aT, bT, a, b, o, s), [A, B], (1, n, m), torch.int32, gpu,
                   what="gemm_int8 aT=%d bT=%d" % (aT, bT))
        both(lambda a, b, r, c, o: ck.gemm_int8_scale(m, k, n, 1, 1, aT, bT, a, b, r, c, True, True, o, s), [A, B, sx[0], sw[0]],
             (1, n, m), torch.half, gpu, what="gemm_int8_scale aT=%d bT=%d" % (aT, bT))
    both(lambda a, r, c, o: ck.gemm_scale(1, n, m, a, r, c, o, True, True, s), [acc, sx[0], sw[0]], (1, n, m), torch.half, gpu, what="gemm_scale")
    Xh = X[0, :, :64].contiguous().view(1, n, 64)
    Wh = W[0, :, :64].contiguous().view(1, m, 64)
    both(lambda a, b, o: ck.gemm_fp16(m, 64, n, 1, 1, True, False, a, b, o, s), [Wh, Xh], (1, n, m), torch.half, gpu, exact=False, what="gemm_fp16")
    # GEMV: 32 vectors against the quantised weights
    vq, vs = qx[0, :32].contiguous(), sx[0, :32].contiguous()
    both(lambda sm, mt, sv, v, o: ck.gemv_broadcast_mat_int8(32, m, k, sm, mt, sv, v, o, s), [sw[0], qw[0], vs, vq], (32, m), torch.half, gpu,
         what="gemv_broadcast_mat_int8")
    both(lambda mt, v, o: ck.gemv_broadcast_mat_fp16(32, m, k, mt, v, o, s), [W[0], X[0, :32].contiguous()], (32, m), torch.half, gpu,
         exact=False, what="gemv_broadcast_mat_fp16")


# (shift 2: buffers that start on an odd element, which the reference's half2 kernels would not take; the kernels here
# move their 16-byte pieces at any address)
@pytest.mark.parametrize("shift", [4, 2])
@pytest.mark.parametrize("shape", [(3, 512, 128), (2, 2048, 64), (4, 100, 72), (2, 600, 250)])
def test_dim1_and_elementwise_unaligned(gpu, shape, shift, monkeypatch):
    _name("layernorm / softmax / elementwise, pointers off 16-byte boundaries", shape, shift)
    monkeypatch.setattr(sys.modules[__name__], "SHIFT_BYTES", shift)
    b, n, m = shape
    g = torch.Generator().manual_seed(32 + n)
    x = (torch.randn(b, n, m, generator=g) * 2).half().to(gpu)
    y = torch.randn(b, n, m, generator=g).half().to(gpu)
    al = (1 + 0.1 * torch.randn(n, generator=g)).half().to(gpu)
    be = (0.1 * torch.randn(n, generator=g)).half().to(gpu)
    mk = (torch.rand(b, m, generator=g) > 0.3).to(torch.int8).to(gpu)
    s = stream()
    both(lambda i, o: ck.layernorm_forward(b, n, m, i, o, 1e-5, True, s), [x], shape, torch.half, gpu, exact=False, what="layernorm")
    both(lambda i, o: ck.softmax_forward(b, n, m, i, o, s), [x], shape, torch.half, gpu, exact=False, what="softmax")
    # (the 8-wide and the element-wise code of gelu may round the last bit differently: a 1e-3 kernel)
    both(lambda i, o: ck.gelu_forward(b, n * m, i, o, s), [x], shape, torch.half, gpu, exact=False, what="gelu")
    both(lambda i, j, o: ck.arith_element_add(b, n * m, i, j, o, s), [x, y], shape, torch.half, gpu, what="element_add")
    both(lambda i, a, c, o: ck.arith_ln_mul_add(b, n, m, i, a, c, o, s), [x, al, be], shape, torch.half, gpu, what="ln_mul_add")
    both(lambda i, k_, o: ck.mask(b, n, m, i, k_, float("-inf"), o, s), [x, mk], shape, torch.half, gpu, what="mask")
    both(lambda i, o: ck.transpose(b, n, m, i, o, s), [x], (b, m, n), torch.half, gpu, what="transpose")
    p = torch.softmax(x.float(), dim=1).half()
    both(lambda o_, g_, o: ck.softmax_backward(b, n, m, o_, g_, o, s), [p, y], shape, torch.half, gpu, exact=False, what="softmax_backward")
    # one-pass quantisers: scale and int8 through one call each
    sc = both(lambda i, o: ck.gemm_calc_scale_transpose(b, n, m, i, o, s), [x], (b, m), torch.half, gpu, what="calc_scale_transpose")
    both(lambda i, c, o: ck.gemm_round_transpose(b, n, m, i, c, o, s), [x, sc], shape, torch.int8, gpu, what="round_transpose")
    for tr in (False, True):
        q_a = torch.zeros((b, m, n) if tr else shape, dtype=torch.int8, device=gpu); s_a = torch.zeros((b, m), dtype=torch.half, device=gpu)
        ck.gemm_quantize_cols(b, n, m, x.data_ptr(), s_a.data_ptr(), q_a.data_ptr(), tr, s)
        xs, q_s, s_s = shifted(x), shifted(torch.zeros_like(q_a)), shifted(torch.zeros_like(s_a))
        ck.gemm_quantize_cols(b, n, m, xs.data_ptr(), s_s.data_ptr(), q_s.data_ptr(), tr, s)
        assert_bits_equal(to_np(s_s), to_np(s_a), "quantize_cols scales (transposed=%s)" % tr)
        assert_bits_equal(to_np(q_s), to_np(q_a), "quantize_cols int8 (transposed=%s)" % tr)


def test_results_do_not_depend_on_timing(gpu):
    """The team kernels add their partial sums in part order and the many-tile softmax hands tiles
    out dynamically: neither may show in the results.  Each kernel runs five times on the same
    input, with other work queued in between, and every run must reproduce the first bit for bit."""
    _name("repeatability")
    g = torch.Generator().manual_seed(41)
    s = stream()
    x = (torch.randn(8, 4096, 512, generator=g) * 2).half().to(gpu)            # teams of 4 (layernorm), 8 (column quantiser)
    sm = (torch.randn(64, 1024, 1024, generator=g) * 3).half().to(gpu)         # 1024 tiles on 256 persistent workgroups
    W = torch.randint(-127, 128, (10240, 4096), generator=g, dtype=torch.int8).to(gpu)
    v = torch.randint(-127, 128, (32, 4096), generator=g, dtype=torch.int8).to(gpu)
    sW = (torch.rand(10240, generator=g) * 0.01 + 1e-3).half().to(gpu); sv = (torch.rand(32, generator=g) * 0.05 + 1e-3).half().to(gpu)
    Wh = torch.randn(2048, 4096, generator=g).half().to(gpu); vh = torch.randn(32, 4096, generator=g).half().to(gpu)
    noise = torch.empty(64 << 20, dtype=torch.half, device=gpu)

    def runs(fn, outs):
        first = None
        for i in range(5):
            for o in outs:
                o.fill_(0)
            if i % 2:
                noise.normal_()          # other kernels ahead of it in the queue
            fn()
            got = [to_np(o).copy() for o in outs]
            if first is None:
                first = got
            else:
                for a, b in zip(got, first):
                    assert_bits_equal(a, b, "run %d differs from run 0" % i)

    y = torch.empty_like(x)
    runs(lambda: ck.layernorm_forward(8, 4096, 512, x.data_ptr(), y.data_ptr(), 1e-5, True, s), [y])
    sc = torch.empty((8, 512), dtype=torch.half, device=gpu); q = torch.empty((8, 512, 4096), dtype=torch.int8, device=gpu)
    runs(lambda: ck.gemm_quantize_cols(8, 4096, 512, x.data_ptr(), sc.data_ptr(), q.data_ptr(), True, s), [sc, q])
    so = torch.empty_like(sm)
    runs(lambda: ck.softmax_forward(64, 1024, 1024, sm.data_ptr(), so.data_ptr(), s), [so])
    tall = sm.view(8, 8192, 1024); to = torch.empty_like(tall)
    runs(lambda: ck.softmax_forward(8, 8192, 1024, tall.data_ptr(), to.data_ptr(), s), [to])
    runs(lambda: ck.softmax_backward(8, 8192, 1024, tall.data_ptr(), tall.data_ptr(), to.data_ptr(), s), [to])
    o = torch.empty((32, 10240), dtype=torch.half, device=gpu)
    runs(lambda: ck.gemv_broadcast_mat_int8(32, 10240, 4096, sW.data_ptr(), W.data_ptr(), sv.data_ptr(), v.data_ptr(), o.data_ptr(), s), [o])
    o2 = torch.empty((32, 2048), dtype=torch.half, device=gpu)
    runs(lambda: ck.gemv_broadcast_mat_fp16(32, 2048, 4096, Wh.data_ptr(), vh.data_ptr(), o2.data_ptr(), s), [o2])


def test_team_launches_overlapping_on_eight_streams(gpu):
    """Team kernels of different kinds queued on eight streams at once, nine rounds of them: each
    launch gets packet slots of its own, so every result equals the single-stream result bit for
    bit and no wait runs out.  The reference's kernels keep no state between launches
    (cuda/layernorm.cu:6-71, cuda/softmax.cu:6-43), so callers may overlap them freely."""
    _name("eight streams of team kernels")
    from cpm_kernels_amd.library import cpmk
    g = torch.Generator().manual_seed(43)
    s0 = stream()
    xs = [(torch.randn(8, 4096, 512, generator=g) * (1 + i)).half().to(gpu) for i in range(8)]
    tall = [(torch.randn(2, 8192, 256, generator=g) * 3).half().to(gpu) for i in range(8)]
    cpmk.async_status()                                         # nothing pending from earlier tests

    def one(i, x, t, s):
        y = torch.empty_like(x); so = torch.empty_like(t)
        sc = torch.empty((8, 512), dtype=torch.half, device=gpu); q = torch.empty((8, 512, 4096), dtype=torch.int8, device=gpu)
        if i % 3 == 0:
            ck.layernorm_forward(8, 4096, 512, x.data_ptr(), y.data_ptr(), 1e-5, True, s)
            ck.softmax_forward(2, 8192, 256, t.data_ptr(), so.data_ptr(), s)
            ck.gemm_quantize_cols(8, 4096, 512, x.data_ptr(), sc.data_ptr(), q.data_ptr(), True, s)
        elif i % 3 == 1:
            ck.softmax_forward(2, 8192, 256, t.data_ptr(), so.data_ptr(), s)
            ck.gemm_quantize_cols(8, 4096, 512, x.data_ptr(), sc.data_ptr(), q.data_ptr(), True, s)
            ck.layernorm_forward(8, 4096, 512, x.data_ptr(), y.data_ptr(), 1e-5, True, s)
        else:
            ck.gemm_quantize_cols(8, 4096, 512, x.data_ptr(), sc.data_ptr(), q.data_ptr(), True, s)
            ck.layernorm_forward(8, 4096, 512, x.data_ptr(), y.data_ptr(), 1e-5, True, s)
            ck.softmax_forward(2, 8192, 256, t.data_ptr(), so.data_ptr(), s)
        return y, so, sc, q

    ref = [one(0, xs[i], tall[i], s0) for i in range(8)]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream() for _ in range(8)]
    for rnd in range(9):
        got = []
        for i, st in enumerate(streams):
            with torch.cuda.stream(st):
                got.append(one(i + rnd, xs[i], tall[i], st.cuda_stream))
        torch.cuda.synchronize()
        cpmk.async_status()                                     # raises if any wait ran out
        for i in range(8):
            for a, b, what in zip(got[i], ref[i], ("layernorm", "softmax", "column scales", "column int8")):
                assert_bits_equal(to_np(a), to_np(b), "round %d stream %d %s" % (rnd, i, what))


def test_more_launches_than_the_pool_holds(gpu):
    """300 tall layernorms back to back on two streams take more packet slots than the pool has, so
    slots are reused while earlier launches may still run: the later launch must wait for the
    earlier one's completion, and all results stay equal."""
    _name("packet pool wraps around")
    from cpm_kernels_amd.library import cpmk
    g = torch.Generator().manual_seed(44)
    x = torch.randn(8, 4096, 512, generator=g).half().to(gpu)
    ref = torch.empty_like(x)
    ck.layernorm_forward(8, 4096, 512, x.data_ptr(), ref.data_ptr(), 1e-5, True, stream())
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream() for _ in range(2)]
    outs = [torch.zeros_like(x) for _ in range(6)]
    for i in range(300):
        st = streams[i % 2]
        with torch.cuda.stream(st):
            ck.layernorm_forward(8, 4096, 512, x.data_ptr(), outs[i % 6].data_ptr(), 1e-5, True, st.cuda_stream)
    torch.cuda.synchronize()
    cpmk.async_status()
    for o in outs:
        assert torch.equal(o.view(torch.int16), ref.view(torch.int16))


def test_a_wait_that_runs_out_is_reported(gpu):
    """A workgroup that gives up waiting sets the device's status word and its mirror in pinned host
    memory.  From then on every call into the library raises the RuntimeError the reference raises
    for any failed launch or synchronisation (library/cudart.py:325-327) -- no caller has to ask --
    until cpmk_async_status has reported the condition once, which clears it.  The self-test kernel
    waits 2 ms for a packet nobody posts and then ends normally."""
    _name("time-out status")
    from cpm_kernels_amd.library import cpmk
    import cpm_kernels_amd
    torch.cuda.synchronize()
    cpmk.async_status()
    x = torch.randn(2, 4096, 64).half().to(gpu); y = torch.empty_like(x); z = torch.empty_like(x)
    ck.layernorm_forward(2, 4096, 64, x.data_ptr(), y.data_ptr(), 1e-5, True, stream())      # (sets the pool up: the mirror exists from here on)
    torch.cuda.synchronize()
    cpmk.selftest_exchange_timeout(2000, stream())
    torch.cuda.synchronize()
    # the next call, whichever it is, reports the failure (its own launch is still made) ...
    with pytest.raises(RuntimeError, match="gave up waiting"):
        ck.gelu_forward(1, 64, x.data_ptr(), z.data_ptr(), stream())
    with pytest.raises(RuntimeError, match="gave up waiting"):
        ck.layernorm_forward(2, 4096, 64, x.data_ptr(), z.data_ptr(), 1e-5, True, stream())
    # ... until the status call has taken it
    with pytest.raises(RuntimeError, match="gave up waiting"):
        cpm_kernels_amd.check()
    cpmk.async_status()                                         # cleared by the read
    # the pool still works afterwards
    ck.layernorm_forward(2, 4096, 64, x.data_ptr(), z.data_ptr(), 1e-5, True, stream())
    assert torch.equal(y.view(torch.int16), z.view(torch.int16)) and bool(torch.isfinite(y).all())
    cpmk.async_status()


def test_captured_team_launch_between_eager_launches_on_another_stream(gpu):
    """A tall layernorm recorded into a HIP graph keeps packet slots that no other launch is ever given,
    so its replays may run while eager team launches on a second stream go round the ring of slots
    (200 launches of 256 slots wrap the 32768-slot ring): every replay and every eager result equals
    the single-stream result bit for bit, and no wait runs out."""
    _name("captured layernorm replayed beside 200 eager team launches on a second stream")
    from cpm_kernels_amd.library import cpmk
    g = torch.Generator().manual_seed(45)
    xa = torch.randn(8, 4096, 512, generator=g).half().to(gpu)
    xb = (torch.randn(8, 4096, 512, generator=g) * 2 + 0.5).half().to(gpu)
    ref_a, ref_b = torch.empty_like(xa), torch.empty_like(xb)
    ck.layernorm_forward(8, 4096, 512, xa.data_ptr(), ref_a.data_ptr(), 1e-5, True, stream())
    ck.layernorm_forward(8, 4096, 512, xb.data_ptr(), ref_b.data_ptr(), 1e-5, True, stream())
    torch.cuda.synchronize()
    cpmk.async_status()
    left = cpmk.exchange_capture_slots_left()
    ya = torch.zeros_like(xa)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ck.layernorm_forward(8, 4096, 512, xa.data_ptr(), ya.data_ptr(), 1e-5, True, stream())
    assert cpmk.exchange_capture_slots_left() == left - 256, "a recorded team launch takes its slots from the capture reserve"
    sa, sb = torch.cuda.Stream(), torch.cuda.Stream()
    outs = [torch.zeros_like(xb) for _ in range(4)]
    for rnd in range(4):
        ya.fill_(0)
        torch.cuda.synchronize()
        for i in range(50):
            with torch.cuda.stream(sb):
                ck.layernorm_forward(8, 4096, 512, xb.data_ptr(), outs[i % 4].data_ptr(), 1e-5, True, sb.cuda_stream)
            if i % 10 == 5:
                with torch.cuda.stream(sa):
                    graph.replay()
        torch.cuda.synchronize()
        cpmk.async_status()
        assert_bits_equal(to_np(ya), to_np(ref_a), "replays of round %d" % rnd)
        for o in outs:
            assert_bits_equal(to_np(o), to_np(ref_b), "eager launches of round %d" % rnd)


def test_captured_many_tile_softmax_beside_eager_ones_on_another_stream(gpu):
    """The many-tile softmax hands its tiles out from two counters in device memory.  They belong to the launch
    (they come out of the exchange pool like a team's packet slots), so a recorded softmax may be replayed while
    any number of eager ones run on a second stream: every result equals the single-stream result bit for bit."""
    _name("captured many-tile softmax replayed beside 120 eager ones on a second stream")
    from cpm_kernels_amd.library import cpmk
    g = torch.Generator().manual_seed(46)
    shape = (40, 1024, 1024)                # 640 column tiles: more than two per compute unit
    xa = (torch.randn(shape, generator=g) * 3).half().to(gpu)
    xb = (torch.randn(shape, generator=g) * 2 + 0.5).half().to(gpu)
    ref_a, ref_b = torch.empty_like(xa), torch.empty_like(xb)
    ck.softmax_forward(*shape, xa.data_ptr(), ref_a.data_ptr(), stream())
    ck.softmax_forward(*shape, xb.data_ptr(), ref_b.data_ptr(), stream())
    torch.cuda.synchronize()
    left = cpmk.exchange_capture_slots_left()
    ya = torch.zeros_like(xa)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ck.softmax_forward(*shape, xa.data_ptr(), ya.data_ptr(), stream())
    assert cpmk.exchange_capture_slots_left() < left, "the recorded launch's counters come out of the capture reserve"
    sa, sb = torch.cuda.Stream(), torch.cuda.Stream()
    outs = [torch.zeros_like(xb) for _ in range(3)]
    for rnd in range(3):
        ya.fill_(0)
        torch.cuda.synchronize()
        for i in range(40):
            with torch.cuda.stream(sb):
                ck.softmax_forward(*shape, xb.data_ptr(), outs[i % 3].data_ptr(), sb.cuda_stream)
            if i % 8 == 4:
                with torch.cuda.stream(sa):
                    graph.replay()
        torch.cuda.synchronize()
        cpmk.async_status()
        assert_bits_equal(to_np(ya), to_np(ref_a), "replays of round %d" % rnd)
        for o in outs:
            assert_bits_equal(to_np(o), to_np(ref_b), "eager launches of round %d" % rnd)
