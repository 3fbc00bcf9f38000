"""GPU parity of the training-side and helper kernels (backward passes, the rest of arith,
transpose, decode-loop utilities) through the C ABI against oracle/training.py.

Bars: bit-exact for the fp16 elementwise family, int8 rounding with its scales, transposes and
copies; results that sum many fp32 terms are compared with the float64 value within
|a - e| <= 2e-3*|e| + atol (the reference's own fp32 block reductions use yet another summation
order), atol stated at each check.
"""
import numpy as np
import pytest
import torch

from oracle import training as ot
import cpm_kernels_amd.kernels as ck
from util import stream, to_gpu, to_np, assert_bits_equal, assert_close_fp16, rand_half

pytestmark = pytest.mark.gpu


def _name(*a):
    print("case", *a, flush=True)


_KEEP = []


def dev(a):
    """Device copy that stays alive until the test module is done with it: a temporary passed as
    `dev(a).data_ptr()` would be freed, and its memory reused, before the kernel runs."""
    t = to_gpu(a)
    _KEEP.append(t)
    if len(_KEEP) > 64:
        torch.cuda.synchronize()
        del _KEEP[:32]
    return t


def _empty(shape, gpu, dtype=torch.half):
    return torch.empty(shape, dtype=dtype, device=gpu)


def special_halves(rng, shape):
    """Random fp16 bit patterns: every exponent incl. subnormals, infinities and NaNs."""
    return rng.integers(0, 65536, size=shape, dtype=np.uint16).view(np.float16)


def assert_fp16_equal_nan_ok(actual, expected, what):
    """Bit equality except that any NaN matches any NaN (payloads are not part of the contract)."""
    a = np.asarray(actual); e = np.asarray(expected)
    assert a.shape == e.shape
    both_nan = np.isnan(a) & np.isnan(e)
    assert_bits_equal(np.where(both_nan, np.float16(0), a), np.where(both_nan, np.float16(0), e), what)


# (the last three: many rows of few columns -- the rows dealt to groups of lanes --, a ragged last piece, a wide tensor)
@pytest.mark.parametrize("shape", [(3, 64), (16, 4096), (1, 2), (5, 1026), (1000, 72), (130, 5002), (8, 1 << 21)])
def test_arith_batch_family(gpu, shape):
    _name("arith batch_*", shape)
    b, n = shape
    rng = np.random.default_rng(b * 7919 + n)
    for trial, gen in enumerate((lambda s: rand_half(rng, s), lambda s: special_halves(rng, s))):
        x, y = gen((b, n)), gen((b, n))
        alpha, beta = gen((n,)), gen((n,))
        xd, yd, ad, bd = map(to_gpu, (x, y, alpha, beta))
        out = _empty((b, n), gpu)
        ck.arith_element_mul(b, n, xd.data_ptr(), yd.data_ptr(), out.data_ptr(), stream())
        assert_fp16_equal_nan_ok(to_np(out), ot.arith_element_mul(x, y), "element_mul %d" % trial)
        ck.arith_batch_add_forward(b, n, xd.data_ptr(), ad.data_ptr(), out.data_ptr(), stream())
        assert_fp16_equal_nan_ok(to_np(out), ot.arith_batch_add_forward(x, alpha), "batch_add_forward %d" % trial)
        ck.arith_batch_mul_add(b, n, xd.data_ptr(), ad.data_ptr(), bd.data_ptr(), out.data_ptr(), stream())
        assert_fp16_equal_nan_ok(to_np(out), ot.arith_batch_mul_add(x, alpha, beta), "batch_mul_add %d" % trial)
        ck.arith_batch_mul(b, n, xd.data_ptr(), ad.data_ptr(), out.data_ptr(), stream())
        assert_fp16_equal_nan_ok(to_np(out), ot.arith_batch_mul(x, alpha), "batch_mul %d" % trial)
        for scale in (0.125, 1.0 / 3.0, 1024.0):
            ck.arith_global_scale(b * n, xd.data_ptr(), scale, out.data_ptr(), stream())
            assert_fp16_equal_nan_ok(to_np(out), ot.arith_global_scale(x, scale), "global_scale %d" % trial)
    # in place
    x = rand_half(rng, (b, n)); alpha = rand_half(rng, (n,))
    xd = to_gpu(x); ad = to_gpu(alpha)
    ck.arith_batch_mul(b, n, xd.data_ptr(), ad.data_ptr(), xd.data_ptr(), stream())
    assert_bits_equal(to_np(xd), ot.arith_batch_mul(x, alpha), "batch_mul in place")
    # column sums
    g = rand_half(rng, (b, n))
    grad = _empty((n,), gpu)
    ck.arith_batch_add_backward(b, n, dev(g).data_ptr(), grad.data_ptr(), stream())
    assert_close_fp16(to_np(grad), ot.arith_batch_add_backward(g), rtol=2e-3, atol=2e-3, what="batch_add_backward")


@pytest.mark.parametrize("shape", [(2, 64, 32), (3, 17, 10), (1, 4096, 64), (2, 5, 1000)])
def test_arith_ln_family(gpu, shape):
    _name("arith ln_*", shape)
    b, n, m = shape
    rng = np.random.default_rng(b * 7919 + n * 31 + m)
    for trial, gen in enumerate((lambda s: rand_half(rng, s), lambda s: special_halves(rng, s))):
        x = gen((b, n, m)); alpha, beta = gen((n,)), gen((n,))
        xd, ad, bd = map(to_gpu, (x, alpha, beta))
        out = _empty((b, n, m), gpu)
        ck.arith_ln_add(b, n, m, xd.data_ptr(), bd.data_ptr(), out.data_ptr(), stream())
        assert_fp16_equal_nan_ok(to_np(out), ot.arith_ln_add(x, beta), "ln_add %d" % trial)
        ck.arith_ln_div(b, n, m, xd.data_ptr(), ad.data_ptr(), out.data_ptr(), stream())
        assert_fp16_equal_nan_ok(to_np(out), ot.arith_ln_div(x, alpha), "ln_div %d" % trial)
        ck.arith_ln_sub_div(b, n, m, xd.data_ptr(), ad.data_ptr(), bd.data_ptr(), out.data_ptr(), stream())
        assert_fp16_equal_nan_ok(to_np(out), ot.arith_ln_sub_div(x, alpha, beta), "ln_sub_div %d" % trial)
    x = rand_half(rng, (b, n, m)); g = rand_half(rng, (b, n, m))
    grad = _empty((n,), gpu)
    ck.arith_ln_mul_backward(b, n, m, dev(x).data_ptr(), dev(g).data_ptr(), grad.data_ptr(), stream())
    tol = 2e-3 * np.sqrt(b * m)          # 2e-3 of the typical magnitude of a sum of b*m unit terms
    assert_close_fp16(to_np(grad), ot.arith_ln_mul_backward(x, g), rtol=2e-3, atol=tol, what="ln_mul_backward")
    ck.arith_ln_add_backward(b, n, m, dev(g).data_ptr(), grad.data_ptr(), stream())
    assert_close_fp16(to_np(grad), ot.arith_ln_add_backward(g), rtol=2e-3, atol=tol, what="ln_add_backward")


def test_arith_ln_div_every_alpha(gpu):
    """x * fp16(1/alpha) for all 65536 alpha bit patterns and a few x: pins the fp16 reciprocal."""
    _name("ln_div all alphas")
    alpha = np.arange(65536, dtype=np.uint32).astype(np.uint16).view(np.float16)
    rng = np.random.default_rng(5)
    x = np.concatenate([np.ones((1, 65536, 2), np.float16), rand_half(rng, (1, 65536, 2), 3.0)], axis=2)
    out = _empty((1, 65536, 4), gpu)
    ck.arith_ln_div(1, 65536, 4, dev(x).data_ptr(), dev(alpha).data_ptr(), out.data_ptr(), stream())
    assert_fp16_equal_nan_ok(to_np(out), ot.arith_ln_div(x, alpha), "ln_div all alphas")
    beta = rand_half(rng, (65536,), 2.0)
    ck.arith_ln_sub_div(1, 65536, 4, dev(x).data_ptr(), dev(alpha).data_ptr(), dev(beta).data_ptr(), out.data_ptr(),
                        stream())
    assert_fp16_equal_nan_ok(to_np(out), ot.arith_ln_sub_div(x, alpha, beta), "ln_sub_div all alphas")


@pytest.mark.parametrize("shape", [(4, 1000), (32, 4096), (1, 6)])
def test_gelu_backward(gpu, shape):
    _name("gelu_backward", shape)
    b, n = shape
    rng = np.random.default_rng(n)
    x = rand_half(rng, (b, n), 2.5)
    x.ravel()[:6] = np.array([0, -0.0, 5, -5, 4.996, -4.996], np.float16)
    g = rand_half(rng, (b, n))
    grad = _empty((b, n), gpu)
    ck.gelu_backward(b, n, dev(g).data_ptr(), dev(x).data_ptr(), grad.data_ptr(), stream())
    # atol: the derivative's own fp32 evaluation error (~1e-6 relative to values of order 1) on outputs near 0
    assert_close_fp16(to_np(grad), ot.gelu_backward(g, x), rtol=1e-3, atol=1e-5, what="gelu_backward")


# (widths that are not whole 16-byte pieces: multiples of 4, of 2, odd -- the register tiles then move 8, 4 or 2 bytes at a time)
COL_SHAPES = [(2, 64, 64), (3, 17, 100), (1, 1024, 96), (2, 5, 7), (1, 3000, 33), (2, 700, 500), (1, 1100, 250), (2, 513, 1)]


@pytest.mark.parametrize("shape", COL_SHAPES)
def test_softmax_backward(gpu, shape):
    _name("softmax_backward", shape)
    b, n, m = shape
    rng = np.random.default_rng(n * 31 + m)
    z = rng.standard_normal((b, n, m)) * 2
    out = (np.exp(z) / np.exp(z).sum(1, keepdims=True)).astype(np.float16)
    g = rand_half(rng, (b, n, m))
    grad = _empty((b, n, m), gpu)
    ck.softmax_backward(b, n, m, dev(out).data_ptr(), dev(g).data_ptr(), grad.data_ptr(), stream())
    assert_close_fp16(to_np(grad), ot.softmax_backward(out, g), rtol=2e-3, atol=1e-5, what="softmax_backward")


def test_column_kernels_on_buffers_off_16_byte_boundaries(gpu):
    """Every buffer starts 2 bytes (the int8 output 1 byte) past a 16-byte boundary: the register tiles fall back to
    narrower accesses and must give the same bits as on aligned buffers."""
    _name("column kernels, misaligned buffers")
    b, n, m = 2, 600, 72
    rng = np.random.default_rng(77)
    x = rand_half(rng, (b, n, m)); g = rand_half(rng, (b, n, m))
    sx = np.abs(rand_half(rng, (b, n), 0.02)) + np.float16(1e-3)

    def off(arr, dtype=torch.half):
        t = torch.from_numpy(arr).to(gpu)
        buf = torch.zeros(t.numel() + 8, dtype=dtype, device=gpu)
        v = buf[1:1 + t.numel()].view(t.shape)
        v.copy_(t)
        return v

    def blank(shape, dtype=torch.half):
        numel = int(np.prod(shape))
        return torch.zeros(numel + 8, dtype=dtype, device=gpu)[1:1 + numel].view(shape)

    xa, ga = to_gpu(x), to_gpu(g)
    xo, go = off(x), off(g)
    assert xo.data_ptr() % 16 == 2
    for name, call in (
        ("softmax_backward", lambda a, c, o: ck.softmax_backward(b, n, m, a.data_ptr(), c.data_ptr(), o.data_ptr(), stream())),
    ):
        o1, o2 = _empty((b, n, m), gpu), blank((b, n, m))
        call(xa, ga, o1); call(xo, go, o2)
        assert_bits_equal(to_np(o2.contiguous()), to_np(o1), name)
    out1, var1 = _empty((b, n, m), gpu), _empty((b, m), gpu)
    out2, var2 = blank((b, n, m)), blank((b, m))
    ck.layernorm_forward_v(b, n, m, xa.data_ptr(), out1.data_ptr(), var1.data_ptr(), 1e-5, stream())
    ck.layernorm_forward_v(b, n, m, xo.data_ptr(), out2.data_ptr(), var2.data_ptr(), 1e-5, stream())
    assert_bits_equal(to_np(out2.contiguous()), to_np(out1), "forward_v out")
    assert_bits_equal(to_np(var2.contiguous()), to_np(var1), "forward_v var")
    gr1, gr2 = _empty((b, n, m), gpu), blank((b, n, m))
    ck.layernorm_backward_v(b, n, m, xa.data_ptr(), ga.data_ptr(), var1.data_ptr(), gr1.data_ptr(), stream())
    ck.layernorm_backward_v(b, n, m, xo.data_ptr(), go.data_ptr(), var2.data_ptr(), gr2.data_ptr(), stream())
    assert_bits_equal(to_np(gr2.contiguous()), to_np(gr1), "backward_v")
    q1, s1 = _empty((b, n, m), gpu, torch.int8), _empty((b, m), gpu)
    q2, s2 = blank((b, n, m), torch.int8), blank((b, m))
    sxa, sxo = to_gpu(sx), off(sx)
    ck.gemm_backward_scale_round(b, n, m, xa.data_ptr(), sxa.data_ptr(), q1.data_ptr(), s1.data_ptr(), False, stream())
    ck.gemm_backward_scale_round(b, n, m, xo.data_ptr(), sxo.data_ptr(), q2.data_ptr(), s2.data_ptr(), False, stream())
    assert_bits_equal(to_np(q2.contiguous()), to_np(q1), "scale_round int8")
    assert_bits_equal(to_np(s2.contiguous()), to_np(s1), "scale_round scale_y")
    sy = np.abs(rand_half(rng, (b, m), 0.02)) + np.float16(1e-3)
    r1, r2 = _empty((b, n), gpu), blank((b, n))
    sya, syo = to_gpu(sy), off(sy)
    ck.gemm_backward_round_scale(b, n, m, xa.data_ptr(), sya.data_ptr(), q1.data_ptr(), r1.data_ptr(), False, stream())
    ck.gemm_backward_round_scale(b, n, m, xo.data_ptr(), syo.data_ptr(), q2.data_ptr(), r2.data_ptr(), False, stream())
    assert_bits_equal(to_np(q2.contiguous()), to_np(q1), "round_scale int8")
    assert_bits_equal(to_np(r2.contiguous()), to_np(r1), "round_scale scale_x")


def test_softmax_backward_more_teams_than_packet_slots(gpu):
    """4200 x 2 team parts exceed the 8192 packet slots of one launch: the batch then goes out in several
    launches.  The whole result must equal the result of the two halves run on their own, and the first
    and last batch entries must match the oracle."""
    _name("softmax_backward, batch split over launches")
    b, n, m = 4200, 600, 64
    gen = torch.Generator(device="cpu").manual_seed(5)
    out = torch.softmax(torch.randn(b, n, m, generator=gen) * 2, dim=1).half().to(gpu)
    g = torch.randn(b, n, m, generator=gen).half().to(gpu)
    grad = torch.zeros_like(out)
    ck.softmax_backward(b, n, m, out.data_ptr(), g.data_ptr(), grad.data_ptr(), stream())
    halves = torch.zeros_like(out)
    h = b // 2
    ck.softmax_backward(h, n, m, out.data_ptr(), g.data_ptr(), halves.data_ptr(), stream())
    ck.softmax_backward(b - h, n, m, out[h:].data_ptr(), g[h:].data_ptr(), halves[h:].data_ptr(), stream())
    assert_bits_equal(to_np(grad), to_np(halves), "one call == two half calls")
    for sl in (slice(0, 3), slice(b - 3, b), slice(4094, 4098)):
        assert_close_fp16(to_np(grad[sl]), ot.softmax_backward(to_np(out[sl]), to_np(g[sl])), rtol=2e-3, atol=1e-5, what="softmax_backward %s" % (sl,))


@pytest.mark.parametrize("shape", COL_SHAPES)
def test_layernorm_training_kernels(gpu, shape):
    _name("layernorm forward_v/mv backward_v/mv", shape)
    b, n, m = shape
    rng = np.random.default_rng(n * 131 + m)
    x = (rng.standard_normal((b, n, m)) * 1.5 + 0.3).astype(np.float16)
    g = rand_half(rng, (b, n, m))
    xd, gd = to_gpu(x), to_gpu(g)
    eps = 1e-5
    out, var, mean, grad = _empty((b, n, m), gpu), _empty((b, m), gpu), _empty((b, m), gpu), _empty((b, n, m), gpu)

    ck.layernorm_forward_v(b, n, m, xd.data_ptr(), out.data_ptr(), var.data_ptr(), eps, stream())
    o_ref, v_ref = ot.layernorm_forward_v(x, eps)
    assert_close_fp16(to_np(out), o_ref, rtol=1e-3, atol=1e-6, what="forward_v out")
    assert_close_fp16(to_np(var), v_ref, rtol=1e-3, what="forward_v var")
    # the plain forward kernel computes the same normalisation
    out2 = _empty((b, n, m), gpu)
    ck.layernorm_forward(b, n, m, xd.data_ptr(), out2.data_ptr(), eps, False, stream())
    assert_close_fp16(to_np(out), to_np(out2).astype(np.float64), rtol=1e-3, atol=1e-6, what="forward_v vs forward")
    v_dev = to_np(var)
    ck.layernorm_backward_v(b, n, m, xd.data_ptr(), gd.data_ptr(), var.data_ptr(), grad.data_ptr(), stream())
    assert_close_fp16(to_np(grad), ot.layernorm_backward_v(x, g, v_dev), rtol=2e-3, atol=2e-4, what="backward_v")

    ck.layernorm_forward_mv(b, n, m, xd.data_ptr(), out.data_ptr(), mean.data_ptr(), var.data_ptr(), eps, stream())
    o_ref, m_ref, v_ref = ot.layernorm_forward_mv(x, eps)
    assert_close_fp16(to_np(out), o_ref, rtol=1e-3, atol=1e-3, what="forward_mv out")
    assert_close_fp16(to_np(mean), m_ref, rtol=1e-3, atol=1e-4, what="forward_mv mean")
    assert_close_fp16(to_np(var), v_ref, rtol=1e-3, what="forward_mv var")
    m_dev, v_dev = to_np(mean), to_np(var)
    ck.layernorm_backward_mv(b, n, m, xd.data_ptr(), gd.data_ptr(), mean.data_ptr(), var.data_ptr(), grad.data_ptr(), stream())
    assert_close_fp16(to_np(grad), ot.layernorm_backward_mv(x, g, m_dev, v_dev), rtol=2e-3, atol=1e-3, what="backward_mv")


# (rows of at most 2048 columns stay in a wave's registers, one, two or four pieces a lane; ragged ends and waves
# whose rows straddle two batch entries)
@pytest.mark.parametrize("shape", COL_SHAPES + [(2, 256, 4096), (3, 37, 512), (2, 50, 1000), (1, 9, 2048), (2, 11, 1544)])
@pytest.mark.parametrize("bc", [False, True])
def test_gemm_backward_quantisers(gpu, shape, bc):
    _name("gemm_backward_round_scale / scale_round", shape, bc)
    b, n, m = shape
    rng = np.random.default_rng(n * 31 + m + bc)
    x = rand_half(rng, (b, n, m))
    x[0, 0, :] = 0
    x[0, :, 0] = 0
    sy = np.abs(rand_half(rng, (1 if bc else b, m), 0.02)) + np.float16(1e-3)
    sx = np.abs(rand_half(rng, (1 if bc else b, n), 0.02)) + np.float16(1e-3)
    xd = to_gpu(x)
    q = _empty((b, n, m), gpu, torch.int8)
    s_row = _empty((b, n), gpu); s_col = _empty((b, m), gpu)
    ck.gemm_backward_round_scale(b, n, m, xd.data_ptr(), dev(sy).data_ptr(), q.data_ptr(), s_row.data_ptr(), bc, stream())
    q_ref, s_ref = ot.gemm_backward_round_scale(x, sy[0] if bc else sy, bc)
    assert_bits_equal(to_np(s_row), s_ref, "round_scale scale_x")
    assert_bits_equal(to_np(q), q_ref, "round_scale int8")
    ck.gemm_backward_scale_round(b, n, m, xd.data_ptr(), dev(sx).data_ptr(), q.data_ptr(), s_col.data_ptr(), bc, stream())
    q_ref, s_ref = ot.gemm_backward_scale_round(x, sx[0] if bc else sx, bc)
    assert_bits_equal(to_np(s_col), s_ref, "scale_round scale_y")
    assert_bits_equal(to_np(q), q_ref, "scale_round int8")


@pytest.mark.parametrize("cfg", [(32, 128, True, 12, 100, 90), (32, 128, False, 4, 64, 200), (64, 512, True, 3, 17, 9),
                                 (32, 128, True, 16, 1024, 1024), (32, 128, False, 5, 333, 2500), (256, 128, True, 2, 70, 130),
                                 # query rows of whole 16-byte pieces (sums over diagonals): the longest, ragged key rows, one-sided
                                 (32, 128, True, 3, 4096, 130), (32, 128, True, 2, 520, 77), (32, 128, False, 2, 256, 300),
                                 (128, 256, True, 9, 8, 4000)])
def test_position_embedding_backward(gpu, cfg):
    _name("position_embedding_backward", cfg)
    import oracle
    num_buckets, max_distance, bidi, heads, ql, kl = cfg
    rng = np.random.default_rng(ql)
    mapping = oracle.position_embedding_init(num_buckets, max_distance, bidi)
    g = rand_half(rng, (heads, kl, ql))
    grad = _empty((heads, num_buckets), gpu)
    ck.position_embedding_backward(ql, kl, num_buckets, max_distance, heads, dev(mapping).data_ptr(), dev(g).data_ptr(),
                                   grad.data_ptr(), bidi, stream())
    ref = ot.position_embedding_backward(ql, kl, num_buckets, max_distance, mapping, g, bidi)
    assert_close_fp16(to_np(grad), ref, rtol=2e-3, atol=2e-3 * np.sqrt(ql * kl / num_buckets), what="position backward")


@pytest.mark.parametrize("shape", [(4, 64, 96, 50), (2, 17, 1000, 7), (8, 32, 64, 3), (3, 5, 8, 1000)])
def test_embedding_backward(gpu, shape):
    """Both stages as the reference's autograd function drives them (torch/embedding.py:33-76):
    ids sorted over the whole batch, cut into `batch` pieces."""
    _name("embedding_backward", shape)
    batch, seq, hidden, vocab = shape
    rng = np.random.default_rng(seq * 31 + vocab)
    ids = rng.integers(0, vocab, (batch, seq)).astype(np.int32)
    order = np.argsort(ids.ravel(), kind="stable").astype(np.int32).reshape(batch, seq)
    sorted_ids = ids.ravel()[order.ravel()].reshape(batch, seq)
    go = rand_half(rng, (batch * seq, hidden))
    grad = torch.zeros((vocab, hidden), dtype=torch.half, device=gpu)
    aux, aux_idx = _empty((batch, hidden), gpu), _empty((batch,), gpu, torch.int32)
    ck.embedding_backward_stage1(batch, seq, hidden, dev(go).data_ptr(), dev(order).data_ptr(), dev(sorted_ids).data_ptr(),
                                 grad.data_ptr(), aux.data_ptr(), aux_idx.data_ptr(), stream())
    g_ref = np.zeros((vocab, hidden), np.float16)
    aux_ref, idx_ref = ot.embedding_backward_stage1(go, order, sorted_ids, g_ref)
    assert_bits_equal(to_np(aux_idx), idx_ref, "stage1 aux idx")
    assert_bits_equal(to_np(aux), aux_ref, "stage1 aux grad")
    assert_bits_equal(to_np(grad), g_ref, "stage1 grad")
    ck.embedding_backward_stage2(batch, hidden, aux.data_ptr(), aux_idx.data_ptr(), grad.data_ptr(), stream())
    assert_bits_equal(to_np(grad), ot.embedding_backward_stage2(aux_ref, idx_ref, g_ref), "stage2 grad")
    # and the pair is a scatter-add
    full = np.zeros((vocab, hidden), np.float64)
    np.add.at(full, ids.ravel(), go.astype(np.float64))
    assert_close_fp16(to_np(grad), full, rtol=2e-3, atol=2e-2, what="embedding gradient")


@pytest.mark.parametrize("shape", [(2, 64, 64), (3, 17, 100), (1, 1000, 3), (2, 5, 7), (1, 4096, 512), (4, 1, 9),
                                   (2, 72, 40), (1, 200, 136), (3, 8, 1032), (2, 4096, 500), (1, 501, 4090), (1, 77, 33)])
def test_transpose(gpu, shape):
    _name("transpose", shape)
    b, n, m = shape
    rng = np.random.default_rng(n * 31 + m)
    x = special_halves(rng, (b, n, m))
    out = _empty((b, m, n), gpu)
    ck.transpose(b, n, m, dev(x).data_ptr(), out.data_ptr(), stream())
    assert_bits_equal(to_np(out), np.ascontiguousarray(x.transpose(0, 2, 1)), "transpose")


@pytest.mark.parametrize("shape", [(2, 64, 64), (3, 17, 100), (1, 1000, 3), (2, 5, 7), (1, 4096, 512), (4, 1, 9),
                                   (2, 80, 48), (1, 208, 144), (3, 16, 1040), (1, 10240, 4096),
                                   # every pairing of 16-byte, 4-byte and single-byte accesses on the two sides
                                   (2, 4096, 500), (2, 500, 4096), (1, 36, 100), (1, 48, 7), (1, 7, 48), (1, 100, 33)])
def test_transpose_i8(gpu, shape):
    _name("transpose_i8", shape)
    b, n, m = shape
    rng = np.random.default_rng(n * 37 + m)
    x = rng.integers(-128, 128, size=(b, n, m), dtype=np.int8)
    xd = torch.from_numpy(x).to(gpu)
    out = torch.zeros((b, m, n), dtype=torch.int8, device=gpu)
    ck.transpose_i8(b, n, m, xd.data_ptr(), out.data_ptr(), stream())
    assert_bits_equal(to_np(out), np.ascontiguousarray(x.transpose(0, 2, 1)), "transpose_i8")


def test_decode_utilities(gpu):
    _name("utils")
    rng = np.random.default_rng(11)
    arr = torch.arange(10, dtype=torch.int32, device=gpu)
    ck.utils.array_add(arr.data_ptr(), 3, 7, stream())
    ck.utils.array_add(arr.data_ptr(), 9, -2, stream())
    ref = np.arange(10, dtype=np.int32); ref[3] += 7; ref[9] -= 2
    assert_bits_equal(to_np(arr), ref, "array_add")

    for b, n in ((2, 1000), (3, 30000), (1, 7)):
        logits = rand_half(rng, (b, n), 4.0)
        freq = rng.integers(0, 4, (b, n)).astype(np.int32)
        ld = to_gpu(logits)
        ck.utils.adjustify_logits(b, n, ld.data_ptr(), 0.7, 0.25, 0.5, dev(freq).data_ptr(), stream())
        assert_bits_equal(to_np(ld), ot.adjustify_logits(logits, 0.7, 0.25, 0.5, freq), "adjustify_logits")

    for b, old, new in ((3, 100, 250), (2, 1025, 1025), (1, 1, 5), (5, 4096, 4160), (2, 2056, 2056), (3, 8, 24)):
        src = rand_half(rng, (b, old))
        dst0 = rand_half(rng, (b, new))
        dd = to_gpu(dst0)
        ck.utils.copy_extend_buffer(b, old, new, dev(src).data_ptr(), dd.data_ptr(), stream())
        ref = dst0.copy(); ref[:, :old] = src
        assert_bits_equal(to_np(dd), ref, "copy_extend_buffer")

    for b, hid, seq, pos in ((2, 300, 17, 5), (1, 4096, 64, 63), (3, 7, 1, 0)):
        src = rand_half(rng, (b, hid, seq))
        out = _empty((b, hid), gpu)
        ck.utils.copy_pos_hidden(b, hid, seq, pos, dev(src).data_ptr(), out.data_ptr(), stream())
        assert_bits_equal(to_np(out), np.ascontiguousarray(src[:, :, pos]), "copy_pos_hidden")

    for n in (1, 63, 5000, 3_000_001):
        x = rand_half(rng, (n,))
        flag = torch.zeros((1,), dtype=torch.int8, device=gpu)
        ck.has_nan_inf(n, dev(x).data_ptr(), flag.data_ptr(), stream())
        assert to_np(flag)[0] == 0, n
        for bad in (np.inf, -np.inf, np.nan):
            y = x.copy(); y[rng.integers(0, n)] = bad
            flag.zero_()
            ck.has_nan_inf(n, dev(y).data_ptr(), flag.data_ptr(), stream())
            assert to_np(flag)[0] == 1, (n, bad)
