"""Tensors with more than 2^31 elements (and int8 operands beyond 2 GB): the element and byte
offsets inside every kernel must be 64-bit, or unsigned 32-bit where the launcher bounds them.
Inputs are drawn on the GPU; the oracle checks slices at the start, on either side of element
2^31 and at the end, where a wrapped index would read or write the wrong place.  The outputs are
pre-filled with a sentinel so that an element nobody wrote is seen as well.
"""
import numpy as np
import pytest
import torch

import oracle
import cpm_kernels_amd.kernels as ck
from util import stream, to_np, assert_bits_equal, assert_close_fp16

pytestmark = pytest.mark.gpu

TWO31 = 2 ** 31


def _name(*a):
    print("case", *a, flush=True)


def _randn_half(shape, seed, gpu, scale=1.0):
    g = torch.Generator(device=gpu).manual_seed(seed)
    x = torch.empty(shape, dtype=torch.half, device=gpu)
    flat = x.view(-1)
    step = 1 << 28                      # draw in pieces: no fp32 copy of the whole tensor
    for i in range(0, flat.numel(), step):
        n = min(step, flat.numel() - i)
        flat[i:i + n] = (torch.randn(n, generator=g, device=gpu) * scale).half()
    return x


def _spans(total, width):
    """Flat element ranges worth checking: start, around 2^31, end."""
    out = [(0, width)]
    if total > TWO31 + width:
        out.append((TWO31 - width, TWO31 + width))
    out.append((total - width, total))
    return out


def test_elementwise_beyond_2_31_elements(gpu):
    batch, n = 2, 2 ** 30 + 2048
    total = batch * n
    _name("elementwise", batch, n)
    x = _randn_half((batch, n), 11, gpu, 2.0)
    y = _randn_half((batch, n), 12, gpu, 2.0)
    out = torch.full((batch, n), 77.0, dtype=torch.half, device=gpu)
    ck.arith_element_add(batch, n, x.data_ptr(), y.data_ptr(), out.data_ptr(), stream())
    xf, yf, of = x.view(-1), y.view(-1), out.view(-1)
    for a, b in _spans(total, 4096):
        assert_bits_equal(to_np(of[a:b]), oracle.arith_element_add(to_np(xf[a:b])[None], to_np(yf[a:b])[None])[0], "element_add [%d,%d)" % (a, b))
    out.fill_(77.0)
    ck.gelu_forward(batch, n, x.data_ptr(), out.data_ptr(), stream())
    for a, b in _spans(total, 4096):
        # tanh-GELU, 1e-3 relative; atol covers the fp16 subnormal tail for very negative inputs
        assert_close_fp16(to_np(of[a:b]), oracle.gelu_forward(to_np(xf[a:b])[None])[0], rtol=1e-3, atol=1e-6, what="gelu [%d,%d)" % (a, b))
    assert int((of == 77.0).sum()) == 0, "gelu left elements unwritten"


def test_softmax_layernorm_beyond_2_31_elements(gpu):
    b, n, m = 2064, 1024, 1024         # batch 2048 starts at element 2^31
    _name("softmax / layernorm, many tiles", (b, n, m))
    x = _randn_half((b, n, m), 13, gpu, 3.0)
    out = torch.full((b, n, m), 77.0, dtype=torch.half, device=gpu)
    ck.softmax_forward(b, n, m, x.data_ptr(), out.data_ptr(), stream())
    for i in (0, 2047, 2048, b - 1):
        assert_close_fp16(to_np(out[i:i + 1]), oracle.softmax_forward(to_np(x[i:i + 1])), rtol=1e-3, atol=1e-7, max_ulp=2, what="softmax batch %d" % i)
    out.fill_(77.0)
    ck.layernorm_forward(b, n, m, x.data_ptr(), out.data_ptr(), 1e-5, True, stream())
    for i in (0, 2047, 2048, b - 1):
        assert_close_fp16(to_np(out[i:i + 1]), oracle.layernorm_forward(to_np(x[i:i + 1]), 1e-5, True), rtol=1e-3, atol=2e-4, what="layernorm batch %d" % i)
    del out
    # tall columns: teams of workgroups, batch 128 starts at element 2^31 (the same 129 * 2^24 values)
    b, n, m = 129, 8192, 2048
    _name("softmax / layernorm, teams", (b, n, m))
    x = x.view(b, n, m)
    out = torch.full((b, n, m), 77.0, dtype=torch.half, device=gpu)
    ck.layernorm_forward(b, n, m, x.data_ptr(), out.data_ptr(), 1e-5, True, stream())
    for i in (0, 127, 128):
        assert_close_fp16(to_np(out[i:i + 1]), oracle.layernorm_forward(to_np(x[i:i + 1]), 1e-5, True), rtol=1e-3, atol=2e-4, what="tall layernorm batch %d" % i)
    out.fill_(77.0)
    ck.softmax_forward(b, n, m, x.data_ptr(), out.data_ptr(), stream())
    for i in (0, 127, 128):
        assert_close_fp16(to_np(out[i:i + 1]), oracle.softmax_forward(to_np(x[i:i + 1])), rtol=1e-3, atol=1e-7, max_ulp=2, what="tall softmax batch %d" % i)


def test_quantisers_beyond_2_31_elements(gpu):
    b, n, m = 1, 2 ** 20 + 16, 2048    # row 2^20 starts at element 2^31
    _name("row quantiser", (b, n, m))
    x = _randn_half((b, n, m), 14, gpu, 1.5)
    sc = torch.full((b, n), 77.0, dtype=torch.half, device=gpu)
    q = torch.full((b, n, m), 99, dtype=torch.int8, device=gpu)
    ck.gemm_quantize(b, n, m, x.data_ptr(), sc.data_ptr(), q.data_ptr(), False, stream())
    for r0 in (0, 2 ** 20 - 8, n - 16):
        xs = to_np(x[:, r0:r0 + 16])
        s_ref = oracle.gemm_calc_scale(xs)
        assert_bits_equal(to_np(sc[:, r0:r0 + 16]), s_ref, "row scales at %d" % r0)
        assert_bits_equal(to_np(q[:, r0:r0 + 16]), oracle.gemm_round(xs, s_ref), "row int8 at %d" % r0)
    # the two-launch form of the same quantisation, whole tensors compared on the device
    sc2 = torch.full((b, n), 77.0, dtype=torch.half, device=gpu)
    q2 = torch.full((b, n, m), 99, dtype=torch.int8, device=gpu)
    ck.gemm_calc_scale(b, n, m, x.data_ptr(), sc2.data_ptr(), stream())
    ck.gemm_round(b, n, m, x.data_ptr(), sc2.data_ptr(), q2.data_ptr(), stream())
    assert torch.equal(sc2, sc) and torch.equal(q2, q), "calc_scale + round == quantize"
    del q, sc, q2
    # dequantisation of an int32 tensor of the same shape
    g = torch.Generator(device=gpu).manual_seed(18)
    acc = torch.randint(-3000000, 3000000, (b, n, m), generator=g, dtype=torch.int32, device=gpu)
    sy = (torch.rand(m, generator=g, device=gpu) * 0.001 + 1e-5).half()
    o16 = torch.full((b, n, m), 77.0, dtype=torch.half, device=gpu)
    ck.gemm_scale(b, n, m, acc.data_ptr(), sc2.data_ptr(), sy.data_ptr(), o16.data_ptr(), True, True, stream())
    for r0 in (0, 2 ** 20 - 8, n - 16):
        ref = oracle.gemm_scale(to_np(acc[:, r0:r0 + 16]), to_np(sc2[0, r0:r0 + 16]), to_np(sy), True, True)
        assert_bits_equal(to_np(o16[:, r0:r0 + 16]), ref, "gemm_scale rows %d.." % r0)
    del acc, o16, sc2
    # per column, written transposed: batch 128 of 129 x (8192, 2048) starts at element 2^31
    del x
    b, n, m = 129, 8192, 2048
    _name("column quantiser", (b, n, m))
    x = _randn_half((b, n, m), 16, gpu, 1.5)
    for tr in (False, True):
        sc = torch.full((b, m), 77.0, dtype=torch.half, device=gpu)
        q = torch.full((b, m, n) if tr else (b, n, m), 99, dtype=torch.int8, device=gpu)
        ck.gemm_quantize_cols(b, n, m, x.data_ptr(), sc.data_ptr(), q.data_ptr(), tr, stream())
        for i in (0, 127, 128):
            xs = to_np(x[i:i + 1])
            s_ref = oracle.gemm_calc_scale_transpose(xs)
            q_ref = oracle.gemm_round_transpose(xs, s_ref)
            assert_bits_equal(to_np(sc[i:i + 1]), s_ref, "column scales, batch %d" % i)
            want = np.ascontiguousarray(q_ref.transpose(0, 2, 1)) if tr else q_ref
            assert_bits_equal(to_np(q[i:i + 1]), want, "column int8 (transposed=%s), batch %d" % (tr, i))
        del q, sc


def _rows_ref(P, Q, rows):
    """Exact int32 rows of P @ Q^T (K-major operands) for the given row indices."""
    return (P[rows].astype(np.float64) @ Q.astype(np.float64).T).astype(np.int32)


def test_gemm_int8_operand_beyond_2_gib_and_output_beyond_2_31(gpu):
    # a row operand of 2.6 GB: byte offsets of its last rows exceed 2^31
    n, k, m = 40000, 65536, 256
    _name("gemm_int8, operand of %.1f GB" % (n * k / 2 ** 30), (n, k, m))
    g = torch.Generator(device=gpu).manual_seed(15)
    P = torch.randint(-127, 128, (1, n, k), generator=g, dtype=torch.int8, device=gpu)     # kernel "B": (n, k)
    Q = torch.randint(-127, 128, (1, m, k), generator=g, dtype=torch.int8, device=gpu)     # kernel "A" with aT: (m, k)
    out = torch.full((1, n, m), 12345, dtype=torch.int32, device=gpu)
    ck.gemm_int8(m, k, n, 1, 1, True, False, Q.data_ptr(), P.data_ptr(), out.data_ptr(), stream())
    Qn = to_np(Q[0])
    for r0 in (0, 32768 - 8, n - 16):      # row 32768 starts at byte 2^31
        rows = slice(r0, r0 + 16)
        assert_bits_equal(to_np(out[0, rows]), _rows_ref(to_np(P[0, rows]), Qn, slice(None)), "rows %d.." % r0)
    del P, Q, out
    # an int32 product of 2.7e9 elements: the output index crosses 2^31 inside row 52428
    n, k, m = 65536, 128, 40960
    _name("gemm_int8, output of %.1f G elements" % (n * m / 1e9), (n, k, m))
    P = torch.randint(-127, 128, (1, n, k), generator=g, dtype=torch.int8, device=gpu)
    Q = torch.randint(-127, 128, (1, m, k), generator=g, dtype=torch.int8, device=gpu)
    out = torch.full((1, n, m), 12345, dtype=torch.int32, device=gpu)
    ck.gemm_int8(m, k, n, 1, 1, True, False, Q.data_ptr(), P.data_ptr(), out.data_ptr(), stream())
    Qn = to_np(Q[0])
    for r0 in (0, TWO31 // m - 8, n - 16):
        rows = slice(r0, r0 + 16)
        assert_bits_equal(to_np(out[0, rows]), _rows_ref(to_np(P[0, rows]), Qn, slice(None)), "rows %d.." % r0)
    # the fused epilogue writes fp16 at the same indices
    srow = (torch.rand(n, generator=g, device=gpu) * 0.05 + 1e-4).half()
    scol = (torch.rand(m, generator=g, device=gpu) * 0.01 + 1e-5).half()
    del out
    o16 = torch.full((1, n, m), 77.0, dtype=torch.half, device=gpu)
    ck.gemm_int8_scale(m, k, n, 1, 1, True, False, Q.data_ptr(), P.data_ptr(), srow.data_ptr(), scol.data_ptr(),
                       True, True, o16.data_ptr(), stream())
    for r0 in (0, TWO31 // m - 8, n - 16):
        rows = slice(r0, r0 + 16)
        acc = _rows_ref(to_np(P[0, rows]), Qn, slice(None))[None]
        ref = oracle.gemm_scale(acc, to_np(srow[rows]), to_np(scol), True, True)
        assert_bits_equal(to_np(o16[:, rows]), ref, "fused rows %d.." % r0)


def test_batches_beyond_the_grid_limit(gpu):
    """70000 batch entries: more than a grid's y or z dimension holds (65535).  The reference indexes
    the batch with the grid's x dimension and has no such limit (kernels/softmax.py:20,
    kernels/transpose.py:17), so the launchers here split such batches over several launches; entry
    65535 onwards must come out like the rest.  Small odd shapes, which take the general kernels."""
    import test_parity_gpu as tp
    import test_training_gpu as tt
    B = 70000
    _name("batch of", B)
    tp.test_softmax_forward(gpu, (B, 5, 3))
    tp.test_layernorm_forward(gpu, (B, 5, 3), True)
    tp.test_calc_scale_and_round_transpose(gpu, (B, 5, 6))
    tp.test_embedding_and_kv_copy(gpu, (B, 4, 3))
    tt.test_softmax_backward(gpu, (B, 6, 2))
    tt.test_layernorm_training_kernels(gpu, (B, 6, 2))
    tt.test_gemm_backward_quantisers(gpu, (B, 6, 2), False)
    tt.test_transpose(gpu, (B, 3, 5))
    tt.test_transpose_i8(gpu, (B, 3, 5))
    rng = np.random.default_rng(17)
    for aT in (False, True):
        for bT in (False, True):
            tp._gemm_case(gpu, 4, 8, 4, B, B, aT, bT, rng)
    tp._gemm_case(gpu, 4, 8, 4, 1, B, True, False, rng)
    tp._gemm_case(gpu, 4, 8, 4, B, 1, True, False, rng)
    # fp16 product and the per-batch transposed GEMV
    A = rng.standard_normal((B, 2, 4)).astype(np.float16)          # (batch, k, m), aT = False
    Bm = rng.standard_normal((B, 6, 2)).astype(np.float16)         # (batch, n, k), bT = False
    Ad, Bd = torch.from_numpy(A).to(gpu), torch.from_numpy(Bm).to(gpu)
    out = torch.full((B, 6, 4), 77.0, dtype=torch.half, device=gpu)
    ck.gemm_fp16(4, 2, 6, B, B, False, False, Ad.data_ptr(), Bd.data_ptr(), out.data_ptr(), stream())
    ref = np.einsum("bnk,bkm->bnm", Bm.astype(np.float64), A.astype(np.float64)).astype(np.float16)
    assert_close_fp16(to_np(out), ref, rtol=1e-3, atol=1e-3, what="gemm_fp16, batch %d" % B)
    mat = rng.standard_normal((B, 6, 8)).astype(np.float16)        # (batch, dim_in, dim_out)
    vec = rng.standard_normal((B, 6)).astype(np.float16)
    md, vd = torch.from_numpy(mat).to(gpu), torch.from_numpy(vec).to(gpu)
    o2 = torch.full((B, 8), 77.0, dtype=torch.half, device=gpu)
    ck.gemv_fp16_transpose(B, 8, 6, md.data_ptr(), vd.data_ptr(), o2.data_ptr(), stream())
    ref = np.einsum("bko,bk->bo", mat.astype(np.float64), vec.astype(np.float64)).astype(np.float16)
    assert_close_fp16(to_np(o2), ref, rtol=1e-3, atol=1e-3, what="gemv_fp16_transpose, batch %d" % B)


def test_training_and_helper_kernels_beyond_2_31_elements(gpu):
    """The remaining kernels with a per-batch layout, on 129 x (8192, 2048): batch 128 starts at
    element 2^31.  Batches 0, 127 and 128 against the CPU restatements."""
    import oracle.training as ot
    b, n, m = 129, 8192, 2048
    _name("training / helper kernels", (b, n, m))
    s = stream()
    x = _randn_half((b, n, m), 21, gpu, 1.5)
    gsrc = _randn_half((b, n, m), 22, gpu, 1.0)
    out = torch.full((b, n, m), 77.0, dtype=torch.half, device=gpu)
    picks = (0, 127, 128)
    # mask and the layernorm affine
    g = torch.Generator(device=gpu).manual_seed(23)
    mk = (torch.rand((b, m), generator=g, device=gpu) > 0.3).to(torch.int8)
    ck.mask(b, n, m, x.data_ptr(), mk.data_ptr(), float("-inf"), out.data_ptr(), s)
    for i in picks:
        assert_bits_equal(to_np(out[i:i + 1]), oracle.mask(to_np(x[i:i + 1]), to_np(mk[i:i + 1]), float("-inf")), "mask batch %d" % i)
    al = (1 + 0.1 * torch.randn(n, generator=g, device=gpu)).half(); be = (0.1 * torch.randn(n, generator=g, device=gpu)).half()
    out.fill_(77.0)
    ck.arith_ln_mul_add(b, n, m, x.data_ptr(), al.data_ptr(), be.data_ptr(), out.data_ptr(), s)
    for i in picks:
        assert_bits_equal(to_np(out[i:i + 1]), oracle.arith_ln_mul_add(to_np(x[i:i + 1]), to_np(al), to_np(be)), "ln_mul_add batch %d" % i)
    # transposes
    outT = torch.full((b, m, n), 77.0, dtype=torch.half, device=gpu)
    ck.transpose(b, n, m, x.data_ptr(), outT.data_ptr(), s)
    for i in picks:
        assert_bits_equal(to_np(outT[i]), np.ascontiguousarray(to_np(x[i]).T), "transpose batch %d" % i)
    del outT
    q = (x.view(torch.int16) & 0xff).to(torch.int8)          # some bytes
    qT = torch.full((b, m, n), 99, dtype=torch.int8, device=gpu)
    ck.transpose_i8(b, n, m, q.data_ptr(), qT.data_ptr(), s)
    for i in picks:
        assert_bits_equal(to_np(qT[i]), np.ascontiguousarray(to_np(q[i]).T), "transpose_i8 batch %d" % i)
    del q, qT
    # dim-1 reductions of the backward pass (teams of 16 workgroups per 64 columns)
    out.fill_(77.0)
    ck.softmax_forward(b, n, m, x.data_ptr(), out.data_ptr(), s)
    grad = torch.full((b, n, m), 77.0, dtype=torch.half, device=gpu)
    ck.softmax_backward(b, n, m, out.data_ptr(), gsrc.data_ptr(), grad.data_ptr(), s)
    for i in picks:
        assert_close_fp16(to_np(grad[i:i + 1]), ot.softmax_backward(to_np(out[i:i + 1]), to_np(gsrc[i:i + 1])), rtol=2e-3, atol=1e-5, what="softmax_backward batch %d" % i)
    mean = torch.empty((b, m), dtype=torch.half, device=gpu); var = torch.empty((b, m), dtype=torch.half, device=gpu)
    ck.layernorm_forward_mv(b, n, m, x.data_ptr(), out.data_ptr(), mean.data_ptr(), var.data_ptr(), 1e-5, s)
    grad.fill_(77.0)
    ck.layernorm_backward_mv(b, n, m, x.data_ptr(), gsrc.data_ptr(), mean.data_ptr(), var.data_ptr(), grad.data_ptr(), s)
    for i in picks:
        o_ref, m_ref, v_ref = ot.layernorm_forward_mv(to_np(x[i:i + 1]), 1e-5)
        assert_close_fp16(to_np(out[i:i + 1]), o_ref, rtol=1e-3, atol=1e-3, what="forward_mv batch %d" % i)
        assert_close_fp16(to_np(mean[i:i + 1]), m_ref, rtol=1e-3, atol=1e-4, what="forward_mv mean, batch %d" % i)
        assert_close_fp16(to_np(grad[i:i + 1]), ot.layernorm_backward_mv(to_np(x[i:i + 1]), to_np(gsrc[i:i + 1]), to_np(mean[i:i + 1]), to_np(var[i:i + 1])),
                          rtol=2e-3, atol=1e-3, what="backward_mv batch %d" % i)


def test_position_bias_rows_longer_than_one_diagonal(gpu):
    """query_len beyond what one LDS diagonal holds (16384 queries): rows are written in pieces, each
    with its own diagonal.  The reference has no such limit (cuda/position_bucket.cu:25-54)."""
    print("case position bias, query_len 40000", flush=True)
    rng = np.random.default_rng(9)
    for (ql, kl, bidi) in ((40000, 19, True), (16385, 33, False), (32768, 5, True)):
        table = oracle.position_embedding_init(32, 128, bidi)
        w = (rng.standard_normal((3, 32)) * 0.02).astype(np.float16)
        td = torch.from_numpy(table).cuda(); wd = torch.from_numpy(w).cuda()
        out = torch.full((3, kl, ql), 7.0, dtype=torch.half, device=gpu)
        ck.position_embedding_forward(ql, kl, 32, 128, 3, td.data_ptr(), wd.data_ptr(), out.data_ptr(), bidi, stream())
        ref = oracle.position_embedding_forward(ql, kl, 32, 128, table, w, bidi)
        assert_bits_equal(to_np(out), ref, "position bias query_len %d" % ql)


def test_general_gemm_with_more_rows_than_a_grid_dimension(gpu):
    """The general (any-shape) product kernels index 64-row tiles with the grid's y dimension: more than
    65535 x 64 output rows go out in several launches.  K = 4 (int8) and 2 (fp16) keep the tensors small;
    rows on either side of the boundary and at the end are compared with exact products."""
    print("case general gemm, 4194340 output rows", flush=True)
    n, m = 65535 * 64 + 100, 4
    g = torch.Generator().manual_seed(12)
    B = torch.randint(-127, 128, (1, n, 4), generator=g, dtype=torch.int8).to(gpu)        # row operand (n, k)
    A = torch.randint(-127, 128, (1, m, 4), generator=g, dtype=torch.int8).to(gpu)        # column operand (m, k)
    out = torch.full((1, n, m), -1, dtype=torch.int32, device=gpu)
    ck.gemm_int8(m, 4, n, 1, 1, True, False, A.data_ptr(), B.data_ptr(), out.data_ptr(), stream())
    ref = (B[0].double() @ A[0].double().t()).to(torch.int32)
    assert torch.equal(out[0], ref)
    Bh = torch.randn(1, n, 2, generator=g).half().to(gpu); Ah = torch.randn(1, m, 2, generator=g).half().to(gpu)
    oh = torch.full((1, n, m), 9.0, dtype=torch.half, device=gpu)
    ck.gemm_fp16(m, 2, n, 1, 1, True, False, Ah.data_ptr(), Bh.data_ptr(), oh.data_ptr(), stream())
    refh = (Bh[0].double() @ Ah[0].double().t())
    for sl in (slice(0, 200), slice(65535 * 64 - 100, 65535 * 64 + 100), slice(n - 50, n)):
        assert_close_fp16(to_np(oh[0, sl]), refh[sl].cpu().numpy(), rtol=1e-3, atol=1e-3, what="general fp16 gemm rows %s" % (sl,))
