"""GPU tests of the torch-level wrappers (cpm_kernels_amd.torch), modelled on the reference's own
test-suite: each wrapper against the torch formulation the reference compares it with
(tests/test_gemm.py, test_layernorm.py, test_softmax.py, test_gelu.py, test_position_embedding.py,
test_mask.py, test_arith.py of the reference), evaluated in fp32 on the CPU, plus the stricter
relations this build adds (fused == kernel-by-kernel, bit for bit).
"""
import numpy as np
import pytest
import torch

import oracle
from oracle import formulations as F
import cpm_kernels_amd.torch as ct
from util import assert_bits_equal, assert_close_fp16, to_np

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _inference_only():
    """Forward results only in this file (gradients: test_torch_backward_gpu.py); no autograd bookkeeping."""
    with torch.no_grad():
        yield


def _name(*a):
    print("case", *a, flush=True)


# shapes after the reference's TEST_CASES (tests/test_gemm.py:43-60): (batch, M, K, N), scaled down
BMM_CASES = [(1, 4, 4, 4), (2, 4, 8, 4), (3, 12, 16, 8), (4, 36, 128, 4), (2, 512, 256, 300),
             (1, 20, 4096, 260), (3, 260, 384, 132)]


@pytest.mark.parametrize("case", BMM_CASES)
@pytest.mark.parametrize("aT", [False, True])
@pytest.mark.parametrize("bT", [False, True])
def test_bmm_int8(gpu, case, aT, bT):
    _name("bmm int8", case, aT, bT)
    batch, M, K, N = case
    g = torch.Generator().manual_seed(M * 31 + K * 7 + N + aT * 2 + bT)
    for bA, bB in ((batch, batch), (1, batch), (batch, 1)):
        A = torch.randn((bA, K, M) if aT else (bA, M, K), generator=g).half()
        B = (torch.randn((bB, N, K) if bT else (bB, K, N), generator=g) * 0.05).half()
        out = ct.bmm(A.cuda(), aT, B.cuda(), bT, int8=True)
        out_unfused = ct.bmm(A.cuda(), aT, B.cuda(), bT, int8=True, fused=False)
        assert out.shape == (batch, M, N) and out.dtype == torch.half
        # the three-launch path equals the reference's six-launch sequence bit for bit
        assert_bits_equal(to_np(out), to_np(out_unfused), "fused bmm == kernel-by-kernel bmm")
        # against the CPU oracle of the same sequence (exact) ...
        Ap = A.transpose(1, 2).contiguous() if aT else A          # (bA, M, K)
        Bp = B.contiguous() if bT else B.transpose(1, 2).contiguous()   # (bB, N, K)
        a_np, b_np = Ap.numpy(), Bp.numpy()
        sa, sb = oracle.gemm_calc_scale(a_np), oracle.gemm_calc_scale(b_np)
        qa, qb = oracle.gemm_round(a_np, sa), oracle.gemm_round(b_np, sb)
        acc = np.einsum("bmk,bnk->bmn", np.broadcast_to(qa, (batch, M, K)).astype(np.float64),
                        np.broadcast_to(qb, (batch, N, K)).astype(np.float64)).astype(np.int32)
        ref = oracle.gemm_scale(acc, np.broadcast_to(sa, (batch, M)).copy(), np.broadcast_to(sb, (batch, N)).copy(),
                                False, False)
        assert_bits_equal(to_np(out), ref, "bmm int8 == oracle sequence")
        # ... and, loosely, against the fp32 fake-quant formulation the reference's test uses
        # (tests/test_gemm.py:87-98 accepts 0.5 absolute; quantising along K as the kernels do)
        loose = F.quant_bmm_rowwise(Ap, Bp).numpy()
        err = np.abs(to_np(out).astype(np.float32) - loose).max()
        assert err < 0.5 and err <= 2e-2 * max(1.0, np.abs(loose).max()), err


# The reference's large TEST_CASES at full size (tests/test_gemm.py:55-59), with its generate_matrix
# (:62-85): batch 8, one side possibly broadcast, each operand possibly stored transposed, values
# randn / k^(1/4) -- drawn from a seed here instead of `random`.  N = 7996 is not a multiple of 8.
BMM_FULL_CASES = [(8, 512, 4096, 2048), (8, 500, 4096, 7996), (8, 512, 10240, 4096), (8, 1024, 512, 4096)]


@pytest.mark.parametrize("case", BMM_FULL_CASES)
def test_bmm_reference_cases_full_size(gpu, case):
    batch, M, K, N = case
    rng = np.random.default_rng(M + 3 * K + 7 * N)
    g = torch.Generator().manual_seed(M * 13 + K * 5 + N)
    for draw in range(2):
        tp = int(rng.integers(0, 3))
        bA, bB = (batch, batch) if tp == 0 else ((1, batch) if tp == 1 else (batch, 1))
        aT, bT = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        _name("bmm full size", case, "draw", draw, "bA", bA, "bB", bB, "aT", aT, "bT", bT)
        skk = K ** 0.25
        a = (torch.randn(bA, M, K, generator=g) / skk).half()              # (bA, M, K)
        b = (torch.randn(bB, N, K, generator=g) / skk).half()              # (bB, N, K): the reference draws (k, n) and transposes; the values are i.i.d. either way
        A = a.transpose(1, 2).contiguous() if aT else a
        B = b if bT else b.transpose(1, 2).contiguous()
        Ad, Bd = A.cuda(), B.cuda()
        out = ct.bmm(Ad, aT, Bd, bT, int8=True)
        assert out.shape == (batch, M, N) and out.dtype == torch.half
        # the oracle's sequence (calc_scale, round, integer product, gemm_scale) on 32 sampled rows of every batch entry
        a_np, b_np = a.numpy(), b.numpy()
        sa, sb = oracle.gemm_calc_scale(a_np), oracle.gemm_calc_scale(b_np)
        qa, qb = oracle.gemm_round(a_np, sa), oracle.gemm_round(b_np, sb)
        rows = np.sort(rng.choice(M, size=32, replace=False))
        got = to_np(out[:, torch.from_numpy(rows).cuda(), :])
        for bi in range(batch):
            ia, ib = (0 if bA == 1 else bi), (0 if bB == 1 else bi)
            acc = (qa[ia, rows].astype(np.float64) @ qb[ib].astype(np.float64).T).astype(np.int32)      # exact: |sum| < 2^53
            ref = oracle.gemm_scale(acc[None], sa[ia:ia + 1, rows].copy(), sb[ib:ib + 1].copy(), False, False)[0]
            assert_bits_equal(got[bi], ref, "bmm int8 full size, batch entry %d" % bi)
        # and the fp16 product of the same operands (int8=False) against float64 on the same rows
        out16 = ct.bmm(Ad, aT, Bd, bT, int8=False)
        got16 = to_np(out16[:, torch.from_numpy(rows).cuda(), :])
        for bi in range(0, batch, 3):
            ia, ib = (0 if bA == 1 else bi), (0 if bB == 1 else bi)
            ref16 = a_np[ia, rows].astype(np.float64) @ b_np[ib].astype(np.float64).T
            assert_close_fp16(got16[bi], ref16, rtol=1e-3, atol=1e-3 * float(np.abs(ref16).max()), what="bmm fp16 full size, batch entry %d" % bi)
        del Ad, Bd, out, out16


@pytest.mark.parametrize("aT", [False, True])
@pytest.mark.parametrize("bT", [False, True])
def test_bmm_fp16(gpu, aT, bT):
    """int8=False: fp16 product with fp32 accumulation (tests/test_gemm.py:62-85 of the reference
    compares with torch.matmul at 5e-2; here 1e-3 against float64)."""
    _name("bmm fp16", aT, bT)
    g = torch.Generator().manual_seed(1 + aT * 2 + bT)
    for (b, M, K, N) in [(2, 8, 16, 12), (3, 130, 256, 64), (1, 512, 512, 260)]:
        A = torch.randn((b, K, M) if aT else (b, M, K), generator=g).half()
        B = (torch.randn((b, N, K) if bT else (b, K, N), generator=g) / K ** 0.5).half()
        out = ct.bmm(A.cuda(), aT, B.cuda(), bT, int8=False)
        ref = F.real_bmm(A.double(), aT, B.double(), bT, False).half()
        assert out.shape == (b, M, N)
        assert_close_fp16(to_np(out), ref.numpy(), rtol=1e-3, atol=1e-3, what="bmm fp16")


@pytest.mark.parametrize("shape", [(4, 512, 64), (3, 100, 40), (2, 4096, 128)])
@pytest.mark.parametrize("bias", [True, False])
def test_layernorm_module(gpu, shape, bias):
    _name("LayerNorm", shape, bias)
    b, n, m = shape
    g = torch.Generator().manual_seed(n + m)
    x = torch.randn(shape, generator=g).half()
    for fused in (True, False):
        ln = ct.LayerNorm(n, eps=1e-5, bias=bias, fused=fused).half().cuda()     # fp16 parameters, as the reference tests use it
        with torch.no_grad():
            ln.weight.copy_((1 + 0.1 * torch.randn(n, generator=g)).half())
            if bias:
                ln.bias.copy_((0.1 * torch.randn(n, generator=g)).half())
        out = ln(x.cuda())
        ref = F.layernorm_dim1(x, ln.weight.cpu(), ln.bias.cpu() if bias else None, 1e-5)
        # reference bar: 5e-3 (tests/test_layernorm.py:100-113); here 1e-3 relative + the fp16
        # rounding of the intermediate (one ulp of an O(1) value) that both implementations carry
        assert_close_fp16(to_np(out), ref.numpy(), rtol=2e-3, atol=2e-3, what="LayerNorm fused=%s" % fused)
        th = ct.LayerNormTH(n, eps=1e-5, bias=bias).half().cuda()
        th.load_state_dict(ln.state_dict())
        assert_close_fp16(to_np(out), to_np(th(x.cuda())), rtol=5e-3, atol=5e-3, what="LayerNorm vs LayerNormTH")
    xi = x.cuda().clone()
    ct.normalize_inplace(xi, 1e-5, True)
    assert_close_fp16(to_np(xi), to_np(ct.normalizeTH(x.cuda(), 1e-5, True)), rtol=2e-3, atol=2e-3, what="normalize_inplace")


@pytest.mark.parametrize("shape", [(8, 128, 256), (3, 77, 40), (2, 1024, 64)])
def test_softmax_wrapper(gpu, shape):
    _name("softmax", shape)
    g = torch.Generator().manual_seed(shape[1])
    x = (torch.randn(shape, generator=g) * 4).half()
    x[:, shape[1] // 2:, 0] = float("-inf")
    out = ct.softmax(x.cuda())
    assert_close_fp16(to_np(out), F.softmax_dim1(x).numpy(), rtol=1e-3, atol=1e-6, what="softmax")
    assert_close_fp16(to_np(out), to_np(ct.softmaxTH(x.cuda())), rtol=2e-3, atol=1e-6, what="softmax vs softmaxTH")
    xi = x.cuda().clone()
    ct.softmax_inplace(xi)
    assert_bits_equal(to_np(xi), to_np(out), "softmax_inplace")


def test_gelu_wrapper(gpu):
    _name("gelu")
    x = (torch.randn(4, 33, 20, generator=torch.Generator().manual_seed(5)) * 3).half()
    out = ct.gelu(x.cuda())
    assert_close_fp16(to_np(out), F.gelu_tanh(x).numpy(), rtol=1e-3, atol=1e-4, what="gelu")
    xi = x.cuda().clone()
    ct.gelu_inplace(xi)
    assert_bits_equal(to_np(xi), to_np(out), "gelu_inplace")


@pytest.mark.parametrize("cfg", [(32, 128, True), (32, 128, False), (64, 256, True), (32, 64, False)])
def test_position_embedding_module(gpu, cfg):
    _name("PositionEmbedding", cfg)
    num_buckets, max_distance, bidi = cfg
    heads = 12
    pe = ct.PositionEmbedding(heads, num_buckets, max_distance, bidi).half().cuda()
    with torch.no_grad():
        pe.weight.copy_((torch.randn(heads, num_buckets, generator=torch.Generator().manual_seed(9)) * 0.02).half())
    out = pe(128, 96)            # (key_len, query_len) as in the reference's forward
    ref = F.position_bias(pe.weight.detach().cpu(), 96, 128, bidi, num_buckets, max_distance)
    assert out.shape == (heads, 128, 96)
    assert_bits_equal(to_np(out), ref.numpy(), "PositionEmbedding")
    th = ct.PositionEmbeddingTH(heads, num_buckets, max_distance, bidi).half().cuda()
    th.load_state_dict(pe.state_dict())
    assert_bits_equal(to_np(th(128, 96)), ref.numpy(), "PositionEmbeddingTH")


def test_mask_and_arith_wrappers(gpu):
    _name("mask/arith")
    g = torch.Generator().manual_seed(3)
    x = torch.randn(3, 16, 40, generator=g).half()
    y = torch.randn(3, 16, 40, generator=g).half()
    mk = torch.rand(3, 40, generator=g) > 0.4
    out = ct.mask(x.cuda(), mk.cuda(), float("-inf"))
    assert_bits_equal(to_np(out), to_np(ct.maskTH(x.cuda(), mk.cuda(), float("-inf"))), "mask")
    assert_bits_equal(to_np(ct.element_add(x.cuda(), y.cuda())), (x + y).numpy(), "element_add")
    al = torch.randn(16, generator=g).half()
    be = torch.randn(16, generator=g).half()
    ref = (x.double() * al.double()[None, :, None] + be.double()[None, :, None]).half()     # fp16 FMA = one rounding
    assert_bits_equal(to_np(ct.ln_mul_add(x.cuda(), al.cuda(), be.cuda())), ref.numpy(), "ln_mul_add")
    assert_bits_equal(to_np(ct.ln_mul(x.cuda(), al.cuda())), (x.double() * al.double()[None, :, None]).half().numpy(), "ln_mul")


def _ffn_block(b, d, dff, s, check):
    """layernorm -> int8 GEMM -> gelu -> int8 GEMM -> residual through the wrappers in the
    reference's native (batch, hidden, seq) layout; the fp32 formulations chained on the CPU for
    the batch entries in `check`.  Returns (device output, reference) restricted to `check`."""
    g = torch.Generator().manual_seed(1004)
    x = torch.randn(b, d, s, generator=g).half()
    W1 = (torch.randn(1, dff, d, generator=g) * 0.02).half()
    W2 = (torch.randn(1, d, dff, generator=g) * 0.02).half()
    ln = ct.LayerNorm(d, eps=1e-5, bias=True).half().cuda()
    with torch.no_grad():
        ln.weight.copy_((1 + 0.1 * torch.randn(d, generator=g)).half())
        ln.bias.copy_((0.1 * torch.randn(d, generator=g)).half())
    xd = x.cuda()
    h = ln(xd)
    h = ct.bmm(W1.cuda(), False, h, False, int8=True)          # (b, dff, s)
    h = ct.gelu(h)
    h = ct.bmm(W2.cuda(), False, h, False, int8=True)          # (b, d, s)
    out = ct.element_add(h, xd)
    # CPU chain in fp32 with the same quantisation axes (weights along K = last dim, activations along K = dim 1)
    xc = x[check]
    r = F.layernorm_dim1(xc, ln.weight.cpu(), ln.bias.cpu(), 1e-5).float()
    def qmm(W, act):   # W (1, N, K), act (b, K, S)
        Wq = F.fake_quant_rows(W.float())
        aq = F.fake_quant_rows(act.transpose(1, 2)).transpose(1, 2)      # per (b, s) column, along K
        return torch.matmul(Wq, aq)
    r = qmm(W1, r).half().float()
    r = F.gelu_tanh(r).half().float()
    r = qmm(W2, r)
    ref = (r + xc.float())
    return to_np(out[check]).astype(np.float32), ref.numpy()


def test_ffn_block_composition(gpu):
    """CPM-2-style FFN block at reduced size against the fp32 formulations.  The tolerance is the
    int8 quantisation noise of two GEMMs."""
    _name("ffn block")
    got, ref = _ffn_block(2, 256, 640, 64, [0, 1])
    err = np.abs(got - ref)
    assert err.max() < 3e-2 and err.mean() < 3e-3, (err.max(), err.mean())


def test_ffn_block_full_size(gpu):
    """The same block at its full size (tokens 8 x 512, 4096 -> 10240 -> 4096); two of the eight
    batch entries are followed on the CPU (entries are independent of each other).  With K = 4096
    and 10240 the quantisation noise of the second product is about 1 % of its output's rms
    (~0.5), hence the absolute bars."""
    _name("ffn block, full size")
    got, ref = _ffn_block(8, 4096, 10240, 512, [0, 5])
    assert np.isfinite(got).all()
    err = np.abs(got - ref)
    rms = float(np.sqrt(np.mean(ref ** 2)))
    print("ffn full size: max err %.4g mean err %.4g output rms %.4g" % (err.max(), err.mean(), rms), flush=True)
    assert err.mean() < 1.5e-2 * rms and err.max() < 0.15 * rms, (err.max(), err.mean(), rms)


def _transformer_layer(b, d, H, dh, dff, s, lens, check, wstd):
    """LayerNorm -> int8 Q/K/V projections -> fp16 scores (B*H, len_k, len_q) + T5 relative bias ->
    padding mask (-inf on padded queries) -> softmax over dim 1 -> fp16 PV -> int8 output
    projection -> residual -> LayerNorm -> int8 FFN with gelu -> residual, through the wrappers
    only in the reference's (batch, hidden, seq) layout, and the same chain of fp32 formulations
    on the CPU for the batch entries in `check`.  Returns (device output[check], reference, probs)."""
    g = torch.Generator().manual_seed(1005)
    x = torch.randn(b, d, s, generator=g).half()
    W = {k: (torch.randn(1, o, i, generator=g) * wstd).half()
         for k, (o, i) in {"q": (d, d), "k": (d, d), "v": (d, d), "o": (d, d), "w1": (dff, d), "w2": (d, dff)}.items()}
    pad = (torch.arange(s)[None, :] < lens[:, None])                     # (b, s) True = real token
    ln1 = ct.LayerNorm(d, bias=True).half().cuda(); ln2 = ct.LayerNorm(d, bias=True).half().cuda()
    pe = ct.PositionEmbedding(H, 32, 128, True).half().cuda()
    for mod in (ln1, ln2):
        mod.weight.copy_((1 + 0.1 * torch.randn(d, generator=g)).half()); mod.bias.copy_((0.1 * torch.randn(d, generator=g)).half())
    pe.weight.copy_((torch.randn(H, 32, generator=g) * 0.02).half())
    Wd = {k: v.cuda() for k, v in W.items()}
    xd, padd = x.cuda(), pad.cuda()

    # ---- device, wrappers only ----
    h = ln1(xd)
    q, k, v = (ct.bmm(Wd[n], False, h, False, int8=True).view(b * H, dh, s) for n in "qkv")
    scores = ct.bmm(k, True, q, False, int8=False)                       # (b*H, s_k, s_q)
    scores = (scores.float() / dh ** 0.5).half()
    bias = pe(s, s)                                                      # (H, s_k, s_q)
    scores = ct.element_add(scores.view(b, H * s * s).contiguous(), bias.reshape(1, -1).expand(b, -1).contiguous())
    scores = ct.mask(scores.view(b, H * s, s), padd, float("-inf"))      # padded queries -> -inf columns
    probs = ct.softmax(scores.view(b * H, s, s))                         # all -inf column -> 0
    ctx = ct.bmm(v, False, probs, False, int8=False).view(b, d, s)       # (b*H, dh, s_q)
    y = ct.element_add(ct.bmm(Wd["o"], False, ctx, False, int8=True), xd)
    h2 = ln2(y)
    f = ct.gelu(ct.bmm(Wd["w1"], False, h2, False, int8=True))
    out = ct.element_add(ct.bmm(Wd["w2"], False, f, False, int8=True), y)

    # ---- CPU, fp32 formulations ----
    def qmm(Wm, act):       # Wm (1, N, K) along K; act (b, K, S) quantised per (b, s) column along K
        # an all-zero column (a padded query after attention) has scale 0: 0/0 in the fp32
        # formulation, 0 in the kernels (NaN -> 0 in the rounding)
        aq = torch.nan_to_num(F.fake_quant_rows(act.float().transpose(1, 2)), nan=0.0).transpose(1, 2)
        return torch.matmul(F.fake_quant_rows(Wm.float()), aq)
    got = to_np(out[check]).astype(np.float32)
    probs_checked = probs.view(b, H, s, s)[check].cpu()
    del q, k, v, scores, probs, ctx, y, h2, f, out, h
    torch.cuda.empty_cache()
    x, pad, b = x[check], pad[check], len(check)
    r = F.layernorm_dim1(x, ln1.weight.cpu(), ln1.bias.cpu(), 1e-5)
    rq, rk, rv = (qmm(W[n], r).half().view(b * H, dh, s).float() for n in "qkv")
    sc = (torch.matmul(rk.transpose(1, 2), rq).half().float() / dh ** 0.5).half().float()
    rb = F.position_bias(pe.weight.cpu(), s, s, True, 32, 128).float()   # (H, s_k, s_q)
    sc = (sc.view(b, H, s, s) + rb[None]).half().float()
    sc = sc.masked_fill(~pad[:, None, None, :], float("-inf")).view(b * H, s, s)
    pr = torch.softmax(sc, dim=1)
    pr = torch.where(torch.isnan(pr), torch.zeros_like(pr), pr).half().float()    # all -inf column -> 0
    rc = torch.matmul(rv, pr).half().view(b, d, s).float()
    ry = (qmm(W["o"], rc).half().float() + x.float()).half()
    r2 = F.layernorm_dim1(ry, ln2.weight.cpu(), ln2.bias.cpu(), 1e-5)
    rf = F.gelu_tanh(qmm(W["w1"], r2).half()).float()
    ref = (qmm(W["w2"], rf).half().float() + ry.float())

    return got, ref.numpy(), probs_checked


def test_transformer_layer_composition(gpu):
    """A CPM-2-shaped transformer layer at reduced size.  The tolerance is the int8 quantisation
    noise of four chained quantised products."""
    _name("transformer layer")
    s = 96
    got, ref, probs = _transformer_layer(2, 256, 4, 64, 640, s, torch.tensor([s, s - 29]), [0, 1], 0.04)
    err = np.abs(got - ref)
    assert np.isfinite(got).all()
    assert err.max() < 6e-2 and err.mean() < 4e-3, (err.max(), err.mean())
    # padded query positions received exactly zero attention
    assert float(probs[1, :, :, s - 29:].abs().max()) == 0.0


def test_transformer_layer_full_size(gpu):
    """The layer at its full size: d_model 4096, 64 heads x 64, d_ff 10240, batch 16, seq 1024,
    lengths drawn from [512, 1024].  The device runs all 16 entries; entry 0 and the shortest
    entry are followed on the CPU (entries are independent).  Bars relative to the output's rms."""
    _name("transformer layer, full size")
    g = torch.Generator().manual_seed(77)
    lens = torch.randint(512, 1025, (16,), generator=g)
    short = int(torch.argmin(lens))
    check = sorted({0, short})
    got, ref, probs = _transformer_layer(16, 4096, 64, 64, 10240, 1024, lens, check, 0.02)
    assert np.isfinite(got).all()
    err = np.abs(got - ref)
    rms = float(np.sqrt(np.mean(ref ** 2)))
    print("layer full size: max err %.4g mean err %.4g output rms %.4g" % (err.max(), err.mean(), rms), flush=True)
    assert err.mean() < 1.5e-2 * rms and err.max() < 0.25 * rms, (err.max(), err.mean(), rms)
    i = check.index(short)
    assert float(probs[i, :, :, int(lens[short]):].abs().max()) == 0.0     # padded queries: exactly zero attention
    # every real query's attention sums to one over the keys
    sums = probs[i, :, :, :int(lens[short])].float().sum(1)
    assert float((sums - 1).abs().max()) < 2e-3
