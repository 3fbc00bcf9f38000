"""Pins oracle/training.py (CPU only) against routes that do not share its formulas:
torch.autograd gradients of independently written forward functions, exact rational arithmetic
for the fp16 elementwise family, numpy scatter-add for the embedding stages.  A dropped term,
a wrong sign or a transposed index in the oracle fails one of these."""
from fractions import Fraction

import numpy as np
import pytest
import torch

import oracle
from oracle import training as ot
from util import assert_bits_equal, rand_half

f16, f64 = np.float16, np.float64


def _close(a, e, rtol, atol, what):
    a = np.asarray(a, f64); e = np.asarray(e, f64)
    assert a.shape == e.shape, what
    assert (np.abs(a - e) <= rtol * np.abs(e) + atol).all(), "%s: max err %g" % (what, np.abs(a - e).max())


def _round_fraction_to_half(q: Fraction) -> np.float16:
    """Correct round-to-nearest-even of an exact rational to fp16, by search over the two neighbours."""
    if q == 0:
        return f16(0)
    lo = f16(float(q))                                   # a candidate close by
    cands = {lo, np.nextafter(lo, f16(np.inf)), np.nextafter(lo, f16(-np.inf))}
    best = None
    for c in cands:
        if not np.isfinite(c):
            continue
        d = abs(Fraction(float(c)) - q)
        key = (d, int(c.view(np.uint16)) & 1)
        if best is None or key < best[0]:
            best = (key, c)
    return best[1]


def test_fp16_elementwise_family_is_singly_rounded():
    rng = np.random.default_rng(0)
    x = rand_half(rng, (2, 6, 4), 3.0); y = rand_half(rng, (2, 6, 4), 3.0)
    alpha = rand_half(rng, (6,), 2.0); beta = rand_half(rng, (6,), 2.0)
    fr = lambda v: Fraction(float(v))                    # noqa: E731
    mul = ot.arith_element_mul(x, y); add = ot.arith_ln_add(x, beta)
    bm = ot.arith_batch_mul_add(x.reshape(12, 4), y[0, 0], y[0, 1])
    for idx in np.ndindex(x.shape):
        assert mul[idx] == _round_fraction_to_half(fr(x[idx]) * fr(y[idx]))
        assert add[idx] == _round_fraction_to_half(fr(x[idx]) + fr(beta[idx[1]]))
    xr = x.reshape(12, 4)
    for i, j in np.ndindex(xr.shape):
        assert bm[i, j] == _round_fraction_to_half(fr(xr[i, j]) * fr(y[0, 0, j]) + fr(y[0, 1, j]))
    # ln_div: the reciprocal is rounded to fp16 before the product (two roundings, not a true quotient)
    div = ot.arith_ln_div(x, alpha)
    for idx in np.ndindex(x.shape):
        r = _round_fraction_to_half(1 / fr(alpha[idx[1]]))
        assert div[idx] == _round_fraction_to_half(fr(x[idx]) * fr(r))
    # ln_sub_div approximates (x - beta) / alpha
    sd = ot.arith_ln_sub_div(x, alpha, beta)
    big = np.abs(alpha) > 0.25
    ref = (x.astype(f64) - beta.astype(f64)[None, :, None]) / alpha.astype(f64)[None, :, None]
    _close(sd[:, big], ref[:, big], 4e-3, 4e-3, "ln_sub_div")
    assert_bits_equal(ot.arith_global_scale(x, 0.5), (x.astype(np.float32) * 0.5).astype(f16), "global_scale")
    assert_bits_equal(ot.arith_batch_add_forward(xr, y[0, 0]), (xr.astype(f64) + y[0, 0].astype(f64)).astype(f16), "batch_add")
    assert_bits_equal(ot.arith_batch_mul(xr, y[0, 0]), (xr.astype(f64) * y[0, 0].astype(f64)).astype(f16), "batch_mul")


def test_sums_are_plain_sums():
    rng = np.random.default_rng(1)
    x = rand_half(rng, (3, 5, 7)); g = rand_half(rng, (3, 5, 7))
    t = torch.from_numpy(x.astype(f64)); tg = torch.from_numpy(g.astype(f64))
    _close(ot.arith_ln_add_backward(g), tg.sum((0, 2)).numpy(), 1e-12, 1e-12, "ln_add_backward")
    _close(ot.arith_ln_mul_backward(x, g), torch.einsum("bnm,bnm->n", t, tg).numpy(), 1e-12, 1e-12, "ln_mul_backward")
    _close(ot.arith_batch_add_backward(g.reshape(15, 7)), tg.reshape(15, 7).sum(0).numpy(), 1e-12, 1e-12, "batch_add_backward")
    # gradient of out = x * alpha[None, :, None] w.r.t. alpha is ln_mul_backward
    alpha = torch.randn(5, dtype=torch.float64, requires_grad=True)
    (t * alpha[None, :, None] * tg).sum().backward()
    _close(ot.arith_ln_mul_backward(x, g), alpha.grad.numpy(), 1e-12, 1e-12, "ln_mul_backward autograd")


def test_gelu_backward_is_the_derivative_of_the_forward_oracle():
    rng = np.random.default_rng(2)
    x = rand_half(rng, (4, 64), 2.0); g = rand_half(rng, (4, 64))
    t = torch.from_numpy(x.astype(f64)).requires_grad_(True)
    y = 0.5 * t * (1 + torch.tanh(0.7978845608028654 * (t + 0.044715 * t ** 3)))
    y.backward(torch.from_numpy(g.astype(f64)))
    # the reference's literals are rounded to 6 digits: agreement to ~1e-5
    _close(ot.gelu_backward(g, x), t.grad.numpy(), 1e-4, 1e-5, "gelu_backward")
    far = np.array([[6.0, -6.0, 5.0, -5.0]], f16)
    assert np.array_equal(ot.gelu_backward(np.ones((1, 4), f16), far), np.array([[1.0, 0.0, 1.0, 0.0]]))


def test_softmax_backward_matches_autograd():
    rng = np.random.default_rng(3)
    z = torch.from_numpy(rng.standard_normal((2, 9, 5))).requires_grad_(True)
    out = torch.softmax(z, dim=1)
    g = rand_half(rng, (2, 9, 5))
    out.backward(torch.from_numpy(g.astype(f64)))
    o16 = out.detach().numpy().astype(f16)
    _close(ot.softmax_backward(o16, g), z.grad.numpy(), 5e-3, 5e-3, "softmax_backward")    # fp16 rounding of `out`
    # exact identity of the formula on the rounded probabilities
    o = o16.astype(f64)
    _close(ot.softmax_backward(o16, g), o * g.astype(f64) - o * (o * g.astype(f64)).sum(1, keepdims=True), 1e-12, 1e-15, "identity")


@pytest.mark.parametrize("rd_mean", [False, True])
def test_layernorm_backward_matches_autograd(rd_mean):
    rng = np.random.default_rng(4)
    x = (rng.standard_normal((2, 24, 6)) * 1.5 + 0.4).astype(f16)
    g = rand_half(rng, (2, 24, 6))
    eps = 1e-5
    t = torch.from_numpy(x.astype(f64)).requires_grad_(True)
    if rd_mean:
        mu = t.mean(1, keepdim=True)
        y = (t - mu) / torch.sqrt(((t - mu) ** 2).mean(1, keepdim=True) + eps)
    else:
        y = t / torch.sqrt((t ** 2).mean(1, keepdim=True) + eps)
    y.backward(torch.from_numpy(g.astype(f64)))
    if rd_mean:
        out, mean, var = ot.layernorm_forward_mv(x, eps)
        _close(out, y.detach().numpy(), 1e-9, 1e-9, "forward_mv")
        # exact statistics -> the analytic gradient; the kernels feed fp16-rounded statistics, so
        # give the oracle statistics that are exact in fp16 by construction of this check's tolerance
        grad = ot.layernorm_backward_mv(x, g, mean.astype(f16), var.astype(f16))
        _close(grad, t.grad.numpy(), 5e-3, 5e-3, "backward_mv")
    else:
        out, var = ot.layernorm_forward_v(x, eps)
        _close(out, y.detach().numpy(), 1e-9, 1e-9, "forward_v")
        grad = ot.layernorm_backward_v(x, g, var.astype(f16))
        _close(grad, t.grad.numpy(), 5e-3, 5e-3, "backward_v")


def test_backward_quantisers_against_scalar_restatement():
    rng = np.random.default_rng(5)
    x = rand_half(rng, (2, 5, 8)); sy = np.abs(rand_half(rng, (2, 8), 0.05)) + f16(0.01)
    sx = np.abs(rand_half(rng, (2, 5), 0.05)) + f16(0.01)
    q, s = ot.gemm_backward_round_scale(x, sy, False)
    for b in range(2):
        for i in range(5):
            p = [np.float32(x[b, i, j]) * np.float32(sy[b, j]) for j in range(8)]
            mx = np.float32(max(abs(v) for v in p) / 127.0)            # float / double literal -> float
            assert s[b, i] == f16(mx)
            for j in range(8):
                assert q[b, i, j] == int(np.rint(np.float32(p[j] / mx)))
    q, s = ot.gemm_backward_scale_round(x, sx[0], True)
    for b in range(2):
        for j in range(8):
            p = [np.float32(x[b, i, j]) * np.float32(sx[0, i]) for i in range(5)]
            mx = np.float32(max(abs(v) for v in p) / 127.0)
            assert s[b, j] == f16(mx)
            for i in range(5):
                assert q[b, i, j] == int(np.rint(np.float32(p[i] / mx)))
    # all-zero row: 0/0 -> 0
    q, s = ot.gemm_backward_round_scale(np.zeros((1, 1, 4), f16), np.ones((1, 4), f16), False)
    assert not q.any() and s[0, 0] == 0


@pytest.mark.parametrize("bidi", [True, False])
def test_position_backward_matches_autograd_of_the_forward_oracle(bidi):
    rng = np.random.default_rng(6)
    nb, md, heads, ql, kl = 32, 128, 3, 40, 50
    mapping = oracle.position_embedding_init(nb, md, bidi)
    # forward oracle on a one-hot-free weight: recover the bucket of every (k, q) from a weight table whose
    # entries are their own bucket index
    w = np.tile(np.arange(nb, dtype=f16), (1, 1))
    bucket = oracle.position_embedding_forward(ql, kl, nb, md, mapping, w, bidi)[0].astype(np.int64)   # (kl, ql)
    g = rand_half(rng, (heads, kl, ql))
    weight = torch.zeros((heads, nb), dtype=torch.float64, requires_grad=True)
    out = weight[:, torch.from_numpy(bucket)]
    out.backward(torch.from_numpy(g.astype(f64)))
    _close(ot.position_embedding_backward(ql, kl, nb, md, mapping, g, bidi), weight.grad.numpy(), 1e-12, 1e-12, "position backward")


def test_embedding_stages_are_a_scatter_add():
    rng = np.random.default_rng(7)
    for batch, seq, hidden, vocab in ((4, 16, 6, 9), (3, 5, 4, 100), (5, 8, 3, 2), (2, 1, 3, 4)):
        ids = rng.integers(0, vocab, (batch, seq)).astype(np.int32)
        order = np.argsort(ids.ravel(), kind="stable").astype(np.int32).reshape(batch, seq)
        sorted_ids = ids.ravel()[order.ravel()].reshape(batch, seq)
        go = rand_half(rng, (batch * seq, hidden))
        grad = np.zeros((vocab, hidden), f16)
        aux, idx = ot.embedding_backward_stage1(go, order, sorted_ids, grad)
        assert np.array_equal(idx, sorted_ids[:, -1])
        ot.embedding_backward_stage2(aux, idx, grad)
        full = np.zeros((vocab, hidden), f64)
        np.add.at(full, ids.ravel(), go.astype(f64))
        _close(grad, full, 3e-3, 1e-2, "embedding backward %s" % ((batch, seq, hidden, vocab),))


def test_adjustify_logits_formula():
    logits = np.array([[1.0, -2.0, 0.5, 8.0]], f16); freq = np.array([[0, 1, 3, 0]], np.int32)
    out = ot.adjustify_logits(logits, 0.5, 0.25, 1.0, freq)
    assert np.array_equal(out, np.array([[2.0, -4.0 - 0.25 - 1.0, 1.0 - 0.75 - 1.0, 16.0]], f16))
