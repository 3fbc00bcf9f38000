"""Pins for the CPU oracle (oracle/cpmk_oracle.c): each restated kernel is checked against
something it does not share code with -- numpy closed forms, exact rational / big-integer
arithmetic, float64 BLAS (exact for these integer products), torch library routines, exhaustive
enumeration over fp16 -- chosen so that a dropped term, a wrong index, a transposed operand or
a wrong rounding fails.  The reference ships no golden vectors for this path
(its tests draw unseeded random inputs); the seeded fixtures under tests/golden/ are made by
tests/golden/make_golden.py from the numpy closed forms, not from the C code.
"""
import math
import os
from fractions import Fraction

import numpy as np
import pytest
import torch

import oracle
from oracle import formulations as F
from util import assert_bits_equal, assert_close_fp16, rand_half

f16, f32, f64 = np.float16, np.float32, np.float64
ALL_H = np.arange(65536, dtype=np.uint16)


# ---------------------------------------------------------------------------------------------
# fp16 conversions
# ---------------------------------------------------------------------------------------------
def test_half_to_float_exhaustive():
    got = oracle.half_to_float(ALL_H)
    ref = ALL_H.view(f16).astype(f32)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))


def test_float_to_half_ties_and_neighbours():
    pos = np.arange(0, 0x7c00, dtype=np.uint16)               # finite non-negative halves
    lo = pos.view(f16).astype(f64)
    hi = (pos + 1).astype(np.uint16).view(f16).astype(f64)
    hi[-1] = 65536.0                                          # successor of 65504 in an unbounded format
    mid = (lo + hi) / 2                                       # exactly representable in fp32 and fp64
    even = np.where(pos % 2 == 0, pos, pos + 1).astype(np.uint16)
    assert np.array_equal(oracle.double_to_half(mid), even)            # ties to even (65520 -> inf)
    assert np.array_equal(oracle.float_to_half(mid.astype(f32)), even)
    eps = np.maximum(mid * 1e-12, 1e-30)
    assert np.array_equal(oracle.double_to_half(mid - eps), pos)       # just below the tie -> down
    assert np.array_equal(oracle.double_to_half(mid + eps), (pos + 1).astype(np.uint16))
    assert np.array_equal(oracle.double_to_half(-mid), even | 0x8000)
    rng = np.random.default_rng(0)
    x = (rng.standard_normal(1 << 20) * 10.0 ** rng.uniform(-9, 5.5, 1 << 20)).astype(f32)
    with np.errstate(over="ignore"):
        assert np.array_equal(oracle.float_to_half(x), x.astype(f16).view(np.uint16))
    sp = np.array([0.0, -0.0, np.inf, -np.inf, 65504.0, 65519.9, 65520.0, 1e-8, 2.0 ** -25, 2.0 ** -24], f64)
    with np.errstate(over="ignore"):
        assert np.array_equal(oracle.double_to_half(sp), sp.astype(f16).view(np.uint16))
    assert (oracle.double_to_half(np.array([np.nan])) & 0x7c00) == 0x7c00


# ---------------------------------------------------------------------------------------------
# scales and rounding
# ---------------------------------------------------------------------------------------------
def np_scale(absmax_f32):
    return (absmax_f32.astype(f32) / f32(127)).astype(f16)


def np_round(x, s):
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        d = x.astype(f32) / s.astype(f32)
        q = np.clip(np.rint(d), -128, 127)
        return np.where(np.isnan(d), 0, q).astype(np.int8)


def test_scale_exhaustive_and_double_divide_equivalence():
    mags = np.arange(0, 0x7c00, dtype=np.uint16).view(f16)          # every finite magnitude
    got = oracle.gemm_calc_scale(mags.reshape(1, -1, 1))[0]
    assert_bits_equal(got, np_scale(mags.astype(f32)), "scale of every fp16 magnitude")
    # the reference divides in double and converts double->float->half (cuda/gemm.cu:74); that
    # equals the single fp32 divide the device uses, for every possible maximum
    via_double = (mags.astype(f64) / 127.0).astype(f32).astype(f16)
    assert_bits_equal(via_double, np_scale(mags.astype(f32)), "double vs float divide")
    assert (np.diff(got.astype(f32)) >= 0).all() and got[0] == 0     # monotone, scale(0) = 0
    neg = (-mags).reshape(1, -1, 1)
    assert_bits_equal(oracle.gemm_calc_scale(neg)[0], got, "absmax uses |x|")


@pytest.mark.parametrize("shape", [(2, 7, 33), (1, 64, 512), (3, 5, 8)])
def test_scale_and_round_closed_forms(shape):
    rng = np.random.default_rng(sum(shape))
    x = rand_half(rng, shape, 1.5)
    x[0, 0] = 0                                       # zero row -> scale 0 -> 0/0 -> 0
    x[0, 1] = (rng.standard_normal(shape[2]) * 1e-5).astype(f16)     # subnormal scale, quotients > 127
    s = oracle.gemm_calc_scale(x)
    assert_bits_equal(s, np_scale(np.abs(x).max(-1).astype(f32)), "calc_scale")
    q = oracle.gemm_round(x, s)
    assert_bits_equal(q, np_round(x, s[..., None]), "round")
    assert (q[0, 0] == 0).all()
    st = oracle.gemm_calc_scale_transpose(x)
    assert_bits_equal(st, np_scale(np.abs(x).max(1).astype(f32)), "calc_scale_transpose")
    assert_bits_equal(oracle.gemm_round_transpose(x, st), np_round(x, st[:, None, :]), "round_transpose")
    # transpose forms == row forms on the transposed tensor
    xt = np.ascontiguousarray(x.transpose(0, 2, 1))
    assert_bits_equal(oracle.gemm_round_transpose(x, st).transpose(0, 2, 1), oracle.gemm_round(xt, st), "T invariant")
    # gemv forms == gemm forms with batch rows
    v = x.reshape(-1, shape[2])
    assert_bits_equal(oracle.gemv_calc_scale(v), s.reshape(-1), "gemv_calc_scale")
    assert_bits_equal(oracle.gemv_round(v, s.reshape(-1)), q.reshape(v.shape), "gemv_round")


def test_round_ties_and_extremes():
    # scale exactly 1.0 (absmax 127): k + 0.5 must round half to even, +-127 stay
    k = np.arange(-126, 127)
    x = np.concatenate([k + 0.5, [127.0, -127.0]]).astype(f16).reshape(1, 1, -1)
    s = oracle.gemm_calc_scale(x)
    assert s[0, 0] == 1.0
    q = oracle.gemm_round(x, s)[0, 0]
    expect = np.concatenate([np.where((k % 2) == 0, k, k + 1), [127, -127]])   # half-even of k+.5
    assert np.array_equal(q, expect)
    # for ordinary rows |q| <= 127 and the absmax element maps to +-127
    rng = np.random.default_rng(1)
    x = rand_half(rng, (1, 200, 300), 1.0)
    q = oracle.gemm_round(x, oracle.gemm_calc_scale(x))
    assert np.abs(q.astype(int)).max() == 127
    am = np.abs(x).argmax(-1)
    assert (np.abs(np.take_along_axis(q, am[..., None], -1)) == 127).all()


def test_round_every_value_against_rational_arithmetic():
    """rint(fp32(x/s)) for every fp16 x and a few scales, against exact rational arithmetic:
    the fp32 rounding of the quotient can never move it onto or across a .5 boundary wrongly."""
    xs = ALL_H.view(f16)
    fin = np.isfinite(xs)
    for sbits in (0x3c00, 0x2e66, 0x1234, 0x0400, 0x03ff, 0x0001):
        s = np.array([sbits], np.uint16).view(f16)
        q = oracle.gemm_round(xs.reshape(1, 1, -1), s.reshape(1, 1))[0, 0]
        sv = Fraction(float(s[0]))
        idx = np.flatnonzero(fin)[:: 37]
        for i in idx:
            d = f32(xs[i]) / f32(s[0])                      # numpy fp32 divide is IEEE
            exact = Fraction(float(xs[i])) / sv
            # d is the fp32 nearest to exact
            assert abs(Fraction(float(d)) - exact) <= abs(Fraction(float(np.nextafter(d, f32(np.inf)))) - exact)
            r = max(-128, min(127, int(np.rint(d))))
            assert q[i] == r


# ---------------------------------------------------------------------------------------------
# int8 GEMM and dequantisation
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("aT", [False, True])
@pytest.mark.parametrize("bT", [False, True])
@pytest.mark.parametrize("bA,bB", [(2, 2), (1, 3), (3, 1)])
def test_gemm_int8_against_float64(aT, bT, bA, bB):
    m, k, n = 12, 20, 8
    rng = np.random.default_rng(m + 2 * k + 3 * n + bA)
    A = rng.integers(-128, 128, (bA, m, k) if aT else (bA, k, m), dtype=np.int8)
    B = rng.integers(-128, 128, (bB, k, n) if bT else (bB, n, k), dtype=np.int8)
    got = oracle.gemm_int8(m, k, n, aT, bT, A, B)
    # independent statement: C[b] = Bop (n,k) @ Aop (k,m) in float64 (exact: k*128^2 < 2^53)
    a_km = A.transpose(0, 2, 1) if aT else A
    b_nk = B.transpose(0, 2, 1) if bT else B
    ref = np.einsum("bjk,bki->bji", np.broadcast_to(b_nk, (max(bA, bB), n, k)).astype(f64),
                    np.broadcast_to(a_km, (max(bA, bB), k, m)).astype(f64))
    assert np.array_equal(got, ref.astype(np.int32))
    assert np.array_equal(oracle.gemm_int8_blas(m, k, n, aT, bT, A, B), got)
    # non-square, asymmetric operands make a swapped or transposed operand fail: spot-check one entry
    b, j, i = max(bA, bB) - 1, n - 1, 1
    av = a_km[0 if bA == 1 else b][:, i].astype(int); bv = b_nk[0 if bB == 1 else b][j].astype(int)
    assert got[b, j, i] == int((av * bv).sum())


def test_gemm_int8_blas_large_k_exact():
    rng = np.random.default_rng(3)
    m, k, n = 24, 4096 + 512, 16
    A = np.full((1, m, k), -128, np.int8); B = np.full((1, n, k), -128, np.int8)
    assert (oracle.gemm_int8_blas(m, k, n, True, False, A, B) == 128 * 128 * k).all()
    A = rng.integers(-128, 128, (1, m, k), dtype=np.int8); B = rng.integers(-128, 128, (1, n, k), dtype=np.int8)
    assert np.array_equal(oracle.gemm_int8_blas(m, k, n, True, False, A, B), oracle.gemm_int8(m, k, n, True, False, A, B))


@pytest.mark.parametrize("bcx,bcy", [(True, True), (False, False), (True, False), (False, True)])
def test_gemm_scale_closed_form(bcx, bcy):
    b, n, m = 3, 9, 14
    rng = np.random.default_rng(5)
    acc = rng.integers(-2 ** 30, 2 ** 30, (b, n, m)).astype(np.int32)
    sx = (rng.random(n if bcx else b * n) * 0.05).astype(f16)
    sy = (rng.random(m if bcy else b * m) * 0.01).astype(f16)
    sxf = (sx.astype(f32)[None, :, None] if bcx else sx.astype(f32).reshape(b, n, 1))
    syf = (sy.astype(f32)[None, None, :] if bcy else sy.astype(f32).reshape(b, 1, m))
    ref = ((acc.astype(f32) * sxf) * syf).astype(f16)          # numpy rounds each fp32 op, then to fp16
    assert_bits_equal(oracle.gemm_scale(acc, sx, sy, bcx, bcy), ref, "gemm_scale")
    if not bcx:
        assert_bits_equal(oracle.gemm_scale_x(acc, sx), (sxf * acc.astype(f32)).astype(f16), "gemm_scale_x")
    if not bcy:
        assert_bits_equal(oracle.gemm_scale_y(acc, sy), (acc.astype(f32) * syf).astype(f16), "gemm_scale_y")


def test_gemv_equals_gemm_path():
    """tests/test_gemv.py:49-59 of the reference pins GEMV == int8 GEMM path at 1e-3; on the same
    quantised operands the two are the same arithmetic, so the oracle must agree bit for bit."""
    rng = np.random.default_rng(8)
    batch, dim_out, dim_in = 5, 28, 44
    mat = rng.integers(-127, 128, (dim_out, dim_in), dtype=np.int8)
    vec = rng.integers(-127, 128, (batch, dim_in), dtype=np.int8)
    sm = (rng.random(dim_out) * 0.01).astype(f16); sv = (rng.random(batch) * 0.05).astype(f16)
    got = oracle.gemv_broadcast_mat_int8(sm, mat, sv, vec)
    acc = oracle.gemm_int8(dim_out, dim_in, batch, True, False, mat[None], vec[None])     # (1, batch, dim_out)
    assert_bits_equal(got, oracle.gemm_scale(acc, sv, sm, True, True)[0], "gemv == gemm path")
    ref = ((vec.astype(f64) @ mat.astype(f64).T).astype(f32) * sv.astype(f32)[:, None] * sm.astype(f32)[None]).astype(f16)
    assert_bits_equal(got, ref, "gemv closed form")


# ---------------------------------------------------------------------------------------------
# layernorm, softmax, gelu
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("rd_mean", [True, False])
def test_layernorm_textbook(rd_mean):
    rng = np.random.default_rng(9)
    x = (rng.standard_normal((3, 257, 20)) * 2 + 0.5).astype(f16)
    eps = 1e-5
    got = oracle.layernorm_forward(x, eps, rd_mean)
    xf = x.astype(f64)
    mean = xf.mean(1, keepdims=True) if rd_mean else 0.0
    var = (xf ** 2).mean(1, keepdims=True) - mean ** 2
    ref = (xf - mean) / np.sqrt(var + eps)
    assert_close_fp16(got, ref.astype(f16), rtol=1e-3, atol=1e-4, what="layernorm textbook")
    g = got.astype(f64)
    if rd_mean:
        assert np.abs(g.mean(1)).max() < 2e-3
    assert np.abs((g ** 2).mean(1) - (1 if rd_mean else (xf ** 2).mean(1) / (var[:, 0] + eps))).max() < 5e-3
    # library cross-check and the m = 1 (contiguous row) case
    th = F.layernorm_dim1(torch.from_numpy(x), torch.ones(257), torch.zeros(257) if rd_mean else None, eps).numpy()
    assert_close_fp16(got, th, rtol=1e-3, atol=1e-4, what="layernorm vs torch formulation")
    row = x[:, :, :1]
    ref1 = torch.nn.functional.layer_norm(torch.from_numpy(row[..., 0]).float(), (257,), eps=eps).numpy() if rd_mean else None
    if rd_mean:
        assert_close_fp16(oracle.layernorm_forward(row, eps, True)[..., 0], ref1.astype(f16), rtol=1e-3, atol=1e-4,
                          what="m=1 == row layer_norm")


def test_softmax_library_and_special_cases():
    rng = np.random.default_rng(10)
    x = rand_half(rng, (2, 100, 12), 4.0)
    x[0, :50, 0] = -np.inf
    x[0, :, 1] = -np.inf
    x[0, :, 2] = -np.inf; x[0, 33, 2] = 3.0
    x[0, :, 3] = f16(2.5)
    got = oracle.softmax_forward(x)
    ref = torch.softmax(torch.from_numpy(x).float(), dim=1).numpy()
    ok = np.ones(x.shape, bool); ok[0, :, 1] = False                  # torch gives NaN for an all -inf column
    assert_close_fp16(got[ok], ref[ok].astype(f16), rtol=1e-3, atol=1e-7, max_ulp=1, what="softmax vs torch")
    assert (got[0, :, 1] == 0).all()                                  # reference: +1e-10 in the sum -> zeros
    assert got[0, 33, 2] == 1.0 and (np.delete(got[0, :, 2], 33) == 0).all()
    assert (got[0, :, 3] == f16(0.01)).all()                          # constant column -> 1/n
    assert np.abs(got.astype(f64).sum(1)[ok[:, 0]] - 1).max() < 2e-3


def test_gelu_exhaustive_against_float64():
    x = ALL_H.view(f16)
    got = oracle.gelu_forward(x)
    xf = x.astype(f64)
    with np.errstate(over="ignore", invalid="ignore"):
        ref = 0.5 * xf * (1.0 + np.tanh(0.7978845608028654 * xf * (1.0 + 0.044715 * xf * xf)))
    fin = np.isfinite(xf)
    # the restatement rounds tanh to fp32 as the reference does, so 1+tanh is quantised to 2^-24
    # for very negative arguments: allow that (atol 1.2e-7 * |x|) on top of one fp16 ulp
    assert_close_fp16(got[fin], ref[fin].astype(f16), rtol=1e-3, atol=4e-6, what="gelu vs float64")
    big = fin & (np.abs(xf) < 3)
    assert_close_fp16(got[big], ref[big].astype(f16), rtol=1e-3, atol=6e-8, max_ulp=1, what="gelu |x|<3")
    assert got[np.flatnonzero(x == f16(np.inf))[0]] == np.inf and np.isnan(got[0x7e00])


# ---------------------------------------------------------------------------------------------
# position buckets
# ---------------------------------------------------------------------------------------------
POS_CONFIGS = [(32, 12, 128, False), (32, 12, 128, True), (32, 24, 256, True), (128, 64, 128, True),
               (16, 64, 256, False), (16, 16, 512, True), (32, 64, 128, True)]


def exact_bucket_table(num_buckets, max_distance, bidirectional):
    """floor(L * log_R(i / E)) + E with big integers: the largest j with R^j * E^L <= i^L."""
    part = num_buckets // (2 if bidirectional else 1)
    E = part // 2
    L = part - E
    R = max_distance // E
    out = []
    for i in range(max_distance):
        if i < E:
            out.append(i)
            continue
        j = 0
        while (R ** (j + 1)) * (E ** L) <= i ** L:
            j += 1
        out.append(j + E)
    return np.array(out, np.int32)


@pytest.mark.parametrize("cfg", POS_CONFIGS)
def test_position_table_and_bias(cfg):
    num_buckets, heads, max_distance, bidi = cfg
    table = oracle.position_embedding_init(num_buckets, max_distance, bidi)
    assert np.array_equal(table, exact_bucket_table(num_buckets, max_distance, bidi))
    part = num_buckets // (2 if bidi else 1)
    assert table.max() <= part - 1 and (np.diff(table) >= 0).all()
    rng = np.random.default_rng(11)
    w = rand_half(rng, (heads, num_buckets))
    for ql, kl in ((128, 128), (40, 300)):
        got = oracle.position_embedding_forward(ql, kl, num_buckets, max_distance, table, w, bidi)
        ref = F.position_bias(torch.from_numpy(w), ql, kl, bidi, num_buckets, max_distance).numpy()
        assert_bits_equal(got, ref, "bias vs HF-T5 formulation %s" % (cfg,))
        assert np.array_equal(got[:, 1:, 1:], got[:, :-1, :-1])            # Toeplitz
        for qp in (0, 17, ql - 1):
            step = oracle.position_embedding_step(qp, kl, num_buckets, max_distance, table, w, bidi)
            assert_bits_equal(step, got[:, :, qp], "step == forward column")


# ---------------------------------------------------------------------------------------------
# fp16 elementwise helpers
# ---------------------------------------------------------------------------------------------
def test_fp16_fma_single_rounding():
    rng = np.random.default_rng(12)
    n = 4000
    x = (rng.standard_normal(n) * 10.0 ** rng.uniform(-4, 3, n)).astype(f16).reshape(1, n, 1)
    a = (rng.standard_normal(n) * 10.0 ** rng.uniform(-3, 2, n)).astype(f16)
    b = (rng.standard_normal(n) * 10.0 ** rng.uniform(-5, 4, n)).astype(f16)
    got = oracle.arith_ln_mul_add(x, a, b).reshape(-1)
    with np.errstate(over="ignore"):
        for i in range(0, n, 3):   # exact rational fma, rounded once
            exact = Fraction(float(x[0, i, 0])) * Fraction(float(a[i])) + Fraction(float(b[i]))
            want = f16(f64(exact)) if abs(exact) < 2 ** 17 else f16(np.inf) * np.sign(float(exact))
            # f64(exact) is exact here (<= 53 significant bits), so numpy's f64->f16 rounds once
            assert got[i] == want or (np.isnan(got[i]) and np.isnan(want)), (i, got[i], want)
        assert_bits_equal(oracle.arith_ln_mul(x, a).reshape(-1), (x.reshape(-1).astype(f32) * a.astype(f32)).astype(f16), "ln_mul")
        y = b.reshape(1, n, 1)
        assert_bits_equal(oracle.arith_element_add(x, y), (x.astype(f64) + y.astype(f64)).astype(f16), "element_add")
    # channel index is dim 1
    x3 = rand_half(rng, (2, 3, 4)); a3 = np.array([1, 2, 3], f16); b3 = np.array([10, 20, 30], f16)
    assert_bits_equal(oracle.arith_ln_mul_add(x3, a3, b3), (x3.astype(f64) * a3[None, :, None] + b3[None, :, None]).astype(f16), "ln_mul_add idx")


def test_mask_closed_form():
    rng = np.random.default_rng(13)
    x = rand_half(rng, (3, 4, 10)); mk = rng.random((3, 10)) < 0.5
    for value in (float("-inf"), 0.0, -1e4, 1e6):
        with np.errstate(over="ignore"):
            ref = np.where(mk[:, None, :], x, f16(value))
        assert_bits_equal(oracle.mask(x, mk, value), ref, "mask %r" % value)
    ref = F.t5_bucket  # noqa: F841  (formulations importable)


# ---------------------------------------------------------------------------------------------
# committed golden fixtures (made from numpy closed forms by tests/golden/make_golden.py)
# ---------------------------------------------------------------------------------------------
def test_oracle_reproduces_golden_fixtures():
    path = os.path.join(os.path.dirname(__file__), "golden", "path_small.npz")
    g = np.load(path)
    assert_bits_equal(oracle.gemm_calc_scale(g["a"]), g["a_scale"], "golden a_scale")
    assert_bits_equal(oracle.gemm_round(g["a"], g["a_scale"]), g["a_q"], "golden a_q")
    assert_bits_equal(oracle.gemm_calc_scale(g["w"]), g["w_scale"], "golden w_scale")
    assert_bits_equal(oracle.gemm_round(g["w"], g["w_scale"]), g["w_q"], "golden w_q")
    M, K = g["a"].shape[1:]; N = g["w"].shape[1]
    acc = oracle.gemm_int8(N, K, M, True, False, g["w_q"], g["a_q"])
    assert np.array_equal(acc, g["acc"])
    assert_bits_equal(oracle.gemm_scale(acc, g["a_scale"], g["w_scale"], True, True), g["out"], "golden out")
    assert_bits_equal(oracle.gemm_calc_scale_transpose(g["a"]), g["a_scale_t"], "golden a_scale_t")
    assert_bits_equal(oracle.gemm_round_transpose(g["a"], g["a_scale_t"]), g["a_q_t"], "golden a_q_t")
    assert_bits_equal(oracle.gemv_broadcast_mat_int8(g["w_scale"][0], g["w_q"][0], g["a_scale"][0], g["a_q"][0]),
                      g["out"][0], "golden gemv == gemm")
    assert np.array_equal(oracle.position_embedding_init(32, 128, True), g["pos_table_32_128_bidi"])
    assert np.array_equal(oracle.position_embedding_init(32, 128, False), g["pos_table_32_128_uni"])
    assert_close_fp16(oracle.layernorm_forward(g["x"], 1e-5, True), g["ln"], rtol=1e-3, atol=1e-4, what="golden ln")
    assert_close_fp16(oracle.softmax_forward(g["x"]), g["softmax"], rtol=1e-3, atol=1e-7, what="golden softmax")
    assert_close_fp16(oracle.gelu_forward(g["x"]), g["gelu"], rtol=1e-3, atol=1e-6, what="golden gelu")


def test_reciprocal_rounding_equals_divide_rounding_exhaustively(tmp_path):
    """The device rounds rows through y = 1/s and one residual step; tests/native/
    recip_round_check.c enumerates all 2^32 (fp16 value, fp16 scale) pairs against the
    divide-then-round of cuda/gemm.cu:16 with the same IEEE operations on the host."""
    import os, shutil, subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    src = os.path.join(os.path.dirname(os.path.abspath(__file__)), "native", "recip_round_check.c")
    exe = str(tmp_path / "recip_round_check")
    subprocess.run(["gcc", "-O2", "-ffp-contract=off", "-mfma", "-msse4.1", "-fopenmp", src, "-o", exe, "-lm"], check=True)
    r = subprocess.run([exe], capture_output=True, text=True)       # the whole grid: seconds on a few cores
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.startswith("4294967296 pairs, 0 mismatches"), r.stdout


def test_short_rounding_of_the_fused_quantisers_exhaustively(tmp_path):
    """The fused quantisers round a row (column) whose scale is a normal fp16 number through
    y = 1/s, one residual step and the low byte of q + 1.5 * 2^23; tests/native/fused_round_check.c
    enumerates every (absmax, x) pair such a row can hold -- about 10^9 -- against the
    divide-then-round of cuda/gemm.cu:16 with the same IEEE operations on the host."""
    import os, shutil, subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    src = os.path.join(os.path.dirname(os.path.abspath(__file__)), "native", "fused_round_check.c")
    exe = str(tmp_path / "fused_round_check")
    subprocess.run(["gcc", "-O2", "-ffp-contract=off", "-mfma", "-msse4.1", "-fopenmp", src, "-o", exe, "-lm"], check=True)
    r = subprocess.run([exe], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.startswith("23568 rows, 989078256 pairs, 0 mismatches"), r.stdout


def test_calc_scale_skips_nan_elements_of_either_kind():
    """cuda/gemm.cu:68-72 takes the maximum with the device's fmaxf, which drops any NaN operand:
    the scale is that of the row with its NaN elements, quiet or signalling, replaced by zeros."""
    rng = np.random.default_rng(3)
    x = (rng.standard_normal((2, 6, 40)) * 3).astype(np.float16)
    b = x.view(np.uint16)
    for (i, j, k, pat) in ((0, 0, 0, 0x7e00), (0, 1, 5, 0x7c01), (1, 2, 39, 0xfdff), (1, 5, 7, 0xffff)):
        b[i, j, k] = pat
    a = np.abs(x.astype(np.float32))
    want = (np.where(np.isnan(a), np.float32(0), a).max(axis=-1) / np.float32(127)).astype(np.float16)
    assert_bits_equal(oracle.gemm_calc_scale(x), want, "row scales with NaN elements")
    xt = np.ascontiguousarray(x.transpose(0, 2, 1))
    assert_bits_equal(oracle.gemm_calc_scale_transpose(xt), want, "column scales with NaN elements")
    q = oracle.gemm_round(x, want)
    assert q[0, 0, 0] == 0 and q[0, 1, 5] == 0 and q[1, 2, 39] == 0 and q[1, 5, 7] == 0
