"""Autograd through the torch wrappers: gradients of every cpm_kernels.torch op against the
plain-torch `TH` formulation of the same op (evaluated in fp32), as the reference's own
tests/test_*.py do.  Tolerances are the reference's (torch.isclose rtol/atol pairs quoted at each
check) or tighter; the int8 product's gradients are additionally checked bit for bit against the
sequence of oracle steps (quantise the gradient, integer product, one-sided dequantisation).
"""
import numpy as np
import pytest
import torch

import oracle
from oracle import training as ot
import cpm_kernels.torch as ct
import cpm_kernels_amd.torch.layernorm as ctl
from util import to_np, assert_bits_equal

pytestmark = pytest.mark.gpu


def _name(*a):
    print("case", *a, flush=True)


def leaf(t):
    return t.clone().detach().requires_grad_(True)


def close(a, b, rtol, atol, what):
    a = a.detach().float(); b = b.detach().float()
    assert a.shape == b.shape, (what, a.shape, b.shape)
    ok = torch.isclose(a, b, rtol, atol)
    assert ok.all(), "%s: %d of %d outside rtol %g atol %g; max abs err %g" % (
        what, int((~ok).sum()), ok.numel(), rtol, atol, float((a - b).abs().max()))


def fake_quant_last(x):
    s = x.abs().amax(dim=-1, keepdim=True) / 127
    return torch.where(s > 0, torch.round(x / s) * s, torch.zeros_like(x))


class StraightThroughQuant(torch.autograd.Function):
    """Forward: per-row absmax fake quantisation along the last dim; backward: identity
    (the comparison function of the reference's tests/test_gemm.py:8-24)."""

    @staticmethod
    def forward(ctx, x):
        return fake_quant_last(x)

    @staticmethod
    def backward(ctx, g):
        return g


def th_bmm(a, aT, b, bT, int8):
    a = a.float().transpose(1, 2) if aT else a.float()          # (b, M, K)
    b = b.float() if bT else b.float().transpose(1, 2)          # (b, N, K)
    if int8:
        a = StraightThroughQuant.apply(a)
        b = StraightThroughQuant.apply(b)
    return torch.matmul(a, b.transpose(1, 2))


BMM_CASES = [(1, 16, 32, 24), (3, 64, 128, 96), (2, 128, 256, 128), (4, 36, 64, 52)]


@pytest.mark.parametrize("case", BMM_CASES)
@pytest.mark.parametrize("aT", [False, True])
@pytest.mark.parametrize("bT", [False, True])
@pytest.mark.parametrize("mode", ["int8", "int8_unfused", "fp16"])
def test_bmm_backward(gpu, case, aT, bT, mode):
    _name("bmm backward", case, aT, bT, mode)
    batch, M, K, N = case
    g = torch.Generator(device="cpu").manual_seed(M * 131 + K + 2 * aT + bT)
    for bcast in (None, "A", "B"):
        if batch == 1 and bcast:
            continue
        bA = 1 if bcast == "A" else batch
        bB = 1 if bcast == "B" else batch
        a = (torch.randn((bA, K, M) if aT else (bA, M, K), generator=g) / K ** 0.25).half().cuda()
        b = (torch.randn((bB, N, K) if bT else (bB, K, N), generator=g) / K ** 0.25).half().cuda()
        grad = (torch.randn((batch, M, N), generator=g) / batch).half().cuda()
        a1, b1, a2, b2 = leaf(a), leaf(b), leaf(a), leaf(b)
        if mode == "fp16":
            out = ct.bmm(a1, aT, b1, bT, False)
        else:
            from cpm_kernels_amd.torch.gemm import bmm
            out = bmm(a1, aT, b1, bT, True, fused=(mode == "int8"))
        ref = th_bmm(a2, aT, b2, bT, mode != "fp16")
        out.backward(gradient=grad)
        ref.backward(gradient=grad.float())
        # relative Frobenius error: rounding the gradient to int8 per row/column costs about 1 %
        for got, want, what in ((a1.grad, a2.grad, "grad_A"), (b1.grad, b2.grad, "grad_B")):
            assert got.shape == want.shape and got.dtype == torch.half
            rel = float((got.float() - want).norm() / want.norm())
            assert rel < (2e-3 if mode == "fp16" else 2.5e-2), (what, bcast, rel)
            # the reference's own bar (tests/test_gemm.py:126-127)
            close(got, want, 5e-1, 5e-1, what)


@pytest.mark.parametrize("aT", [False, True])
@pytest.mark.parametrize("bT", [False, True])
@pytest.mark.parametrize("fused", [False, True])
# (the second case: M and N of at least 128 that are not multiples of 64 -- the fused backward then contracts over
# rows lengthened with zeros)
@pytest.mark.parametrize("dims", [(2, 24, 32, 20), (2, 200, 32, 132)])
def test_bmm_int8_backward_bits(gpu, aT, bT, fused, dims):
    """Every step of GEMMInt8.backward restated with the oracle: bit-identical gradients."""
    _name("bmm int8 backward bits", aT, bT, fused, dims)
    from cpm_kernels_amd.torch.gemm import bmm
    batch, M, K, N = dims
    rng = np.random.default_rng(aT * 2 + bT)
    A = (rng.standard_normal((batch, M, K)) / 2).astype(np.float16)          # logical (M, K)
    B = (rng.standard_normal((batch, N, K)) / 2).astype(np.float16)          # logical (N, K) = B^T
    G = (rng.standard_normal((batch, M, N)) / 2).astype(np.float16)
    a_dev = torch.from_numpy(np.ascontiguousarray(A.transpose(0, 2, 1)) if aT else A).cuda().requires_grad_(True)
    b_dev = torch.from_numpy(B if bT else np.ascontiguousarray(B.transpose(0, 2, 1))).cuda().requires_grad_(True)
    out = bmm(a_dev, aT, b_dev, bT, True, fused=fused)
    out.backward(gradient=torch.from_numpy(G).cuda())
    sA = oracle.gemm_calc_scale(A); qA = oracle.gemm_round(A, sA)
    sB = oracle.gemm_calc_scale(B); qB = oracle.gemm_round(B, sB)
    qGa, sGa = ot.gemm_backward_round_scale(G, sB, False)                    # rows of G scaled by scale_B per column
    accA = np.einsum("bmn,bnk->bmk", qGa.astype(np.int64), qB.astype(np.int64)).astype(np.int32)
    gA = oracle.gemm_scale_x(accA, sGa)                                      # (b, M, K)
    qGb, sGb = ot.gemm_backward_scale_round(G, sA, False)                    # columns of G scaled by scale_A per row
    accB = np.einsum("bmn,bmk->bnk", qGb.astype(np.int64), qA.astype(np.int64)).astype(np.int32)
    gB = oracle.gemm_scale_x(accB, sGb)                                      # (b, N, K)
    assert_bits_equal(to_np(a_dev.grad), np.ascontiguousarray(gA.transpose(0, 2, 1)) if aT else gA, "grad_A")
    assert_bits_equal(to_np(b_dev.grad), gB if bT else np.ascontiguousarray(gB.transpose(0, 2, 1)), "grad_B")


@pytest.mark.parametrize("bias", [True, False])
@pytest.mark.parametrize("shape", [(4, 128, 64), (2, 768, 96), (1, 2048, 80)])
def test_layernorm_backward(gpu, bias, shape):
    _name("LayerNorm backward", bias, shape)
    b, n, m = shape
    torch.manual_seed(n + bias)
    l1 = ct.LayerNorm(n, 1e-5, bias=bias)
    l2 = ct.LayerNormTH(n, 1e-5, bias=bias)
    w = torch.randn(n) * 0.1 + 1
    l1.weight.data = w.clone(); l2.weight.data = w.clone()
    if bias:
        bb = torch.randn(n)
        l1.bias.data = bb.clone(); l2.bias.data = bb.clone()
    l1 = l1.half().cuda(); l2 = l2.cuda()
    x = torch.randn((b, n, m), device="cuda").half()
    x1 = leaf(x); x2 = leaf(x.float())
    y1 = l1(x1); y2 = l2(x2)
    close(y1, y2, 1e-2, 1e-2, "forward")                                     # tests/test_layernorm.py:45
    rd = torch.randn(x.size(), device="cuda").half()
    y1.backward(gradient=rd); y2.backward(gradient=rd.float())
    close(x1.grad, x2.grad, 1e-2, 1e-2, "grad x")                            # :51
    close(l1.weight.grad, l2.weight.grad, 1e-2, 1e-2 * (b * m) ** 0.5, "grad weight")   # reference: 1e-1, 5e-1
    if bias:
        close(l1.bias.grad, l2.bias.grad, 1e-2, 1e-2 * (b * m) ** 0.5, "grad bias")


@pytest.mark.parametrize("shape", [(2, 256, 64), (1, 1536, 72)])
def test_layernorm_ops_with_the_reference_argument_lists(gpu, shape):
    """OpLayerNormMean(x, eps, weight, bias) and OpLayerNormNoMean(x, eps, weight), the reference's two
    autograd functions (torch/layernorm.py:7-156): outputs and every gradient equal to OpLayerNorm's bit
    for bit (they run the same kernels), the right number of gradients for their argument lists, and the
    output against the oracle's layernorm followed by the fp16 affine."""
    _name("OpLayerNormMean / OpLayerNormNoMean", shape)
    b, n, m = shape
    torch.manual_seed(n * 3 + m)
    x = torch.randn(shape, device="cuda").half()
    w = (torch.randn(n, device="cuda") * 0.1 + 1).half()
    bb = (torch.randn(n, device="cuda") * 0.1).half()
    rd = torch.randn(shape, device="cuda").half()
    for mean in (True, False):
        x1, w1, x2, w2 = leaf(x), leaf(w), leaf(x), leaf(w)
        if mean:
            b1, b2 = leaf(bb), leaf(bb)
            y1 = ctl.OpLayerNormMean.apply(x1, 1e-5, w1, b1)
            y2 = ctl.OpLayerNorm.apply(x2, 1e-5, w2, b2, True)
        else:
            y1 = ctl.OpLayerNormNoMean.apply(x1, 1e-5, w1)
            y2 = ctl.OpLayerNorm.apply(x2, 1e-5, w2, None, True)
        assert_bits_equal(to_np(y1), to_np(y2), "forward, mean=%s" % mean)
        norm = oracle.layernorm_forward(to_np(x), 1e-5, mean).astype(np.float32)
        wf = to_np(w).astype(np.float32)[None, :, None]
        exp = norm * wf + (to_np(bb).astype(np.float32)[None, :, None] if mean else 0.0)
        got = to_np(y1).astype(np.float32)
        assert np.all(np.abs(got - exp) <= 2e-3 * np.abs(exp) + 2e-3), "forward against the oracle, mean=%s" % mean
        y1.backward(gradient=rd); y2.backward(gradient=rd)
        assert_bits_equal(to_np(x1.grad), to_np(x2.grad), "grad x, mean=%s" % mean)
        assert_bits_equal(to_np(w1.grad), to_np(w2.grad), "grad weight, mean=%s" % mean)
        if mean:
            assert_bits_equal(to_np(b1.grad), to_np(b2.grad), "grad bias")
        # against the TH formulation in fp32, at test_layernorm_backward's bars
        l2 = ct.LayerNormTH(n, 1e-5, bias=mean).cuda()
        l2.weight.data = w.float().clone()
        if mean:
            l2.bias.data = bb.float().clone()
        x3 = leaf(x.float())
        l2(x3).backward(gradient=rd.float())
        close(x1.grad, x3.grad, 1e-2, 1e-2, "grad x vs TH, mean=%s" % mean)
        close(w1.grad, l2.weight.grad, 1e-2, 1e-2 * (b * m) ** 0.5, "grad weight vs TH, mean=%s" % mean)


@pytest.mark.parametrize("shape", [(2, 128, 64), (3, 1000, 17), (1, 4096, 40)])
def test_softmax_gelu_mask_backward(gpu, shape):
    _name("softmax / gelu / mask backward", shape)
    b, n, m = shape
    torch.manual_seed(n)
    x = torch.randn(shape, device="cuda").half()
    rd = torch.randn(shape, device="cuda").half()
    x1, x2 = leaf(x), leaf(x.float())
    ct.softmax(x1).backward(gradient=rd); ct.softmaxTH(x2).backward(gradient=rd.float())
    close(x1.grad, x2.grad, 1e-3, 1e-3, "softmax grad")                      # tests/test_softmax.py:31
    x1, x2 = leaf(x), leaf(x.float())
    ct.gelu(x1).backward(gradient=rd); ct.geluTH(x2).backward(gradient=rd.float())
    close(x1.grad, x2.grad, 1e-3, 1e-3, "gelu grad")                         # reference bar 1e-2 (tests/test_gelu.py:21)
    mask = torch.rand((b, m), device="cuda") > 0.3
    x1, x2 = leaf(x), leaf(x)
    ct.mask(x1, mask, -1e4).backward(gradient=rd); ct.maskTH(x2, mask, -1e4).backward(gradient=rd)
    assert torch.equal(x1.grad, x2.grad)


def test_arith_backward(gpu):
    _name("arith backward")
    torch.manual_seed(3)
    b, n, m = 3, 96, 50
    x = torch.randn((b, n, m), device="cuda").half(); y = torch.randn((b, n, m), device="cuda").half()
    alpha = (torch.randn(n, device="cuda") * 0.1 + 1).half(); beta = torch.randn(n, device="cuda").half()
    rd = torch.randn((b, n, m), device="cuda").half()

    def run(fn, fn_th, *args):
        a1 = [leaf(t) for t in args]; a2 = [leaf(t.float()) for t in args]
        o1 = fn(*a1); o2 = fn_th(*a2)
        close(o1, o2, 1e-2, 1e-2, fn.__name__)
        o1.backward(gradient=rd); o2.backward(gradient=rd.float())
        for i, (p, q) in enumerate(zip(a1, a2)):
            atol = 1e-2 if p.grad.ndim == 3 else 1e-2 * (b * m) ** 0.5       # channel sums of b*m terms
            close(p.grad, q.grad, 1e-2, atol, "%s grad %d" % (fn.__name__, i))

    run(ct.element_add, ct.element_addTH, x, y)
    run(ct.element_mul, ct.element_mulTH, x, y)
    run(ct.ln_mul_add, ct.ln_mul_addTH, x, alpha, beta)
    run(ct.ln_mul, ct.ln_mulTH, x, alpha)
    run(ct.ln_add, ct.ln_addTH, x, beta)
    run(lambda t: ct.global_scale(t, 0.37), lambda t: ct.global_scaleTH(t, 0.37), x)
    y2 = torch.randn((n, m), device="cuda").half()
    a1, c1, a2, c2 = leaf(x), leaf(y2), leaf(x.float()), leaf(y2.float())
    ct.batched_add(a1, c1).backward(gradient=rd); ct.batched_addTH(a2, c2).backward(gradient=rd.float())
    close(a1.grad, a2.grad, 1e-2, 1e-2, "batched_add grad x"); close(c1.grad, c2.grad, 1e-2, 2e-2, "batched_add grad y")
    # forward-only ops and the in-place forms
    close(ct.ln_div(x, alpha), ct.ln_divTH(x.float(), alpha.float()), 1e-2, 1e-2, "ln_div")
    close(ct.ln_sub_div(x, alpha, beta), ct.ln_sub_divTH(x.float(), alpha.float(), beta.float()), 1e-2, 1e-2, "ln_sub_div")
    for inplace, th, args in ((ct.ln_div_inplace, ct.ln_divTH, (alpha,)), (ct.ln_sub_div_inplace, ct.ln_sub_divTH, (alpha, beta)),
                              (ct.ln_add_inplace, ct.ln_addTH, (beta,)), (ct.element_mul_inplace, ct.element_mulTH, (y,)),
                              (ct.batched_add_inplace, ct.batched_addTH, (y2,)),
                              (ct.global_scale_inplace, ct.global_scaleTH, (0.5,))):
        t = x.clone()
        inplace(t, *args)
        close(t, th(x.float(), *[a.float() if torch.is_tensor(a) else a for a in args]), 1e-2, 1e-2, inplace.__name__)


@pytest.mark.parametrize("cfg", [(32, 128, True, 12, 100, 90), (32, 128, False, 4, 64, 200)])
def test_position_embedding_backward_module(gpu, cfg):
    _name("PositionEmbedding backward", cfg)
    num_buckets, max_distance, bidi, heads, ql, kl = cfg
    torch.manual_seed(ql)
    p1 = ct.PositionEmbedding(heads, num_buckets, max_distance, bidi)
    p2 = ct.PositionEmbeddingTH(heads, num_buckets, max_distance, bidi)
    p2.weight.data = p1.weight.data.clone()
    p1 = p1.half().cuda(); p2 = p2.cuda()
    o1 = p1(kl, ql); o2 = p2(kl, ql)
    close(o1, o2, 1e-3, 1e-3, "forward")
    rd = torch.randn(o1.size(), device="cuda").half()
    o1.backward(gradient=rd); o2.backward(gradient=rd.float())
    close(p1.weight.grad, p2.weight.grad, 2e-3, 2e-3 * (ql * kl / num_buckets) ** 0.5, "weight grad")


@pytest.mark.parametrize("shape", [(4, 64, 96, 50), (2, 17, 1000, 7), (3, 33, 64, 2000)])
def test_embedding_module(gpu, shape):
    _name("Embedding forward/backward", shape)
    batch, seq, hidden, vocab = shape
    torch.manual_seed(seq)
    e1 = ct.Embedding(vocab, hidden); e2 = ct.EmbeddingTH(vocab, hidden)
    w = torch.randn(vocab, hidden).half()
    e1.weight.data = w.clone(); e2.weight.data = w.clone()
    e1 = e1.cuda(); e2 = e2.cuda()
    ids = torch.randint(0, vocab, (batch, seq), dtype=torch.int32, device="cuda")
    o1 = e1(ids); o2 = e2(ids.long())
    assert torch.equal(o1, o2)
    rd = torch.randn(o1.size(), device="cuda").half()
    o1.backward(gradient=rd)
    full = torch.zeros((vocab, hidden), device="cuda", dtype=torch.float32)
    full.index_add_(0, ids.view(-1).long(), rd.float().transpose(1, 2).reshape(-1, hidden))
    close(e1.weight.grad, full, 2e-3, 1e-2, "embedding weight grad")         # reference bar 1e-3/1e-3 on smaller sums


def test_transpose_and_has_nan_inf(gpu):
    _name("transpose / has_nan_inf wrappers")
    torch.manual_seed(1)
    x = torch.randn((3, 50, 70), device="cuda").half()
    x1 = leaf(x)
    o = ct.transpose(x1)
    assert torch.equal(o, ct.transposeTH(x).contiguous())
    rd = torch.randn(o.size(), device="cuda").half()
    o.backward(gradient=rd)
    assert torch.equal(x1.grad, rd.transpose(1, 2).contiguous())
    assert not bool(ct.has_nan_inf(x))
    y = x.clone(); y[1, 2, 3] = float("inf")
    assert bool(ct.has_nan_inf(y))
    flag = torch.zeros(1, dtype=torch.bool, device="cuda")[0]
    y[1, 2, 3] = float("nan")
    ct.has_nan_inf(y, flag)
    assert bool(flag)
