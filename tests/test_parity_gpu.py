"""GPU parity: every HIP kernel, called through the C ABI (cpm_kernels_amd.kernels -> ctypes ->
libcpmk_hip.so), against the CPU oracle on the same seeded inputs.

Bars (from the path's contract): bit-exact for scales, int8 rounding, int32 accumulators,
dequantised outputs (the multiplication order is fixed, so they can be), position buckets,
bias gather and the fp16 elementwise helpers; |a-e| <= 1e-3*|e| + atol for layernorm, softmax
and gelu, with atol stated at each test.
"""
import numpy as np
import pytest
import torch

import oracle
import cpm_kernels_amd.kernels as ck
from util import stream, to_gpu, to_np, assert_bits_equal, assert_close_fp16, rand_half

pytestmark = pytest.mark.gpu


def _name(*a):
    print("case", *a, flush=True)


# ---------------------------------------------------------------------------------------------
# quantisation
# ---------------------------------------------------------------------------------------------
def adversarial_rows(rng, n, m):
    """Rows that stress the rounding contract: zeros, one huge value, subnormal-scale rows,
    exact .5 ties, constant rows, +-max fp16."""
    x = rand_half(rng, (n, m))
    if n >= 8 and m >= 8:
        x[0] = 0
        x[1] = 0; x[1, m // 2] = 65504
        x[2] = (rng.standard_normal(m) * 1e-5).astype(np.float16)          # absmax < 9e-4 -> subnormal scale
        x[3] = np.float16(6e-8)                                            # scale underflows to 0
        # ties: scale = 1/127*127 ... choose absmax 127 -> scale 1.0 exactly, values k+0.5
        x[4] = (rng.integers(-126, 126, m) + 0.5).astype(np.float16); x[4, 0] = 127
        x[5] = np.float16(-3.0)
        x[6] = rand_half(rng, (m,), 100.0); x[6, -1] = -65504
        x[7] = rand_half(rng, (m,), 0.02)
    return x


QUANT_SHAPES = [(1, 512, 4096), (3, 17, 1000), (2, 5, 7), (1, 1, 8), (2, 64, 48), (1, 9, 8200), (4, 33, 16),
                (1, 2100, 128), (1, 3, 20480), (2, 4096, 192), (1, 1032, 72), (3, 520, 8),
                (1, 10240, 192), (2, 16384, 64), (1, 16392, 64),
                # tall columns in widths that are not whole 16-byte pieces (the team kernel, one column at a time)
                (2, 4096, 500), (1, 1040, 77), (1, 2100, 36),
                # rows in registers moving 4 or 2 bytes or one element at a time, up to the longest such rows
                (3, 33, 250), (2, 9, 8190), (1, 5, 8191), (2, 40, 4100)]


@pytest.mark.parametrize("shape", QUANT_SHAPES)
def test_calc_scale_and_round(gpu, shape):
    _name("calc_scale/round", shape)
    b, n, m = shape
    rng = np.random.default_rng(b * 1000003 + n * 1009 + m)
    x = np.stack([adversarial_rows(rng, n, m) for _ in range(b)])
    xd = to_gpu(x)
    sd = torch.empty((b, n), dtype=torch.half, device=gpu)
    ck.gemm_calc_scale(b, n, m, xd.data_ptr(), sd.data_ptr(), stream())
    s_ref = oracle.gemm_calc_scale(x)
    assert_bits_equal(to_np(sd), s_ref, "gemm_calc_scale %s" % (shape,))
    qd = torch.empty((b, n, m), dtype=torch.int8, device=gpu)
    ck.gemm_round(b, n, m, xd.data_ptr(), sd.data_ptr(), qd.data_ptr(), stream())
    assert_bits_equal(to_np(qd), oracle.gemm_round(x, s_ref), "gemm_round %s" % (shape,))
    # fused launcher == the two launches
    s2 = torch.empty_like(sd); q2 = torch.empty_like(qd)
    ck.gemm_quantize(b, n, m, xd.data_ptr(), s2.data_ptr(), q2.data_ptr(), False, stream())
    assert_bits_equal(to_np(s2), s_ref, "gemm_quantize scale")
    assert_bits_equal(to_np(q2), to_np(qd), "gemm_quantize int8")
    # gemv forms are the same arithmetic on (batch*n, m)
    sv = torch.empty((b * n,), dtype=torch.half, device=gpu)
    ck.gemv_calc_scale(b * n, m, xd.data_ptr(), sv.data_ptr(), stream())
    assert_bits_equal(to_np(sv), s_ref.reshape(-1), "gemv_calc_scale")
    qv = torch.empty((b * n, m), dtype=torch.int8, device=gpu)
    ck.gemv_round(b * n, m, xd.data_ptr(), sv.data_ptr(), qv.data_ptr(), stream())
    assert_bits_equal(to_np(qv).reshape(b, n, m), to_np(qd), "gemv_round")


@pytest.mark.parametrize("shape", QUANT_SHAPES)
def test_calc_scale_and_round_transpose(gpu, shape):
    _name("calc_scale_transpose/round_transpose", shape)
    b, n, m = shape
    rng = np.random.default_rng(7 + b * 1000003 + n * 1009 + m)
    # adversarial columns: build on the transposed view
    x = np.stack([np.ascontiguousarray(adversarial_rows(rng, m, n).T) for _ in range(b)])
    xd = to_gpu(x)
    sd = torch.empty((b, m), dtype=torch.half, device=gpu)
    ck.gemm_calc_scale_transpose(b, n, m, xd.data_ptr(), sd.data_ptr(), stream())
    s_ref = oracle.gemm_calc_scale_transpose(x)
    assert_bits_equal(to_np(sd), s_ref, "gemm_calc_scale_transpose %s" % (shape,))
    qd = torch.empty((b, n, m), dtype=torch.int8, device=gpu)
    ck.gemm_round_transpose(b, n, m, xd.data_ptr(), sd.data_ptr(), qd.data_ptr(), stream())
    assert_bits_equal(to_np(qd), oracle.gemm_round_transpose(x, s_ref), "gemm_round_transpose %s" % (shape,))
    s2 = torch.empty_like(sd); q2 = torch.empty_like(qd)
    ck.gemm_quantize(b, n, m, xd.data_ptr(), s2.data_ptr(), q2.data_ptr(), True, stream())
    assert_bits_equal(to_np(s2), s_ref, "gemm_quantize(T) scale")
    assert_bits_equal(to_np(q2), to_np(qd), "gemm_quantize(T) int8")
    # invariant: transposed forms == row forms on the transposed tensor
    xt = np.ascontiguousarray(x.transpose(0, 2, 1))
    assert_bits_equal(s_ref, oracle.gemm_calc_scale(xt), "transpose invariant (scale)")
    # one-pass column quantiser, int8 in place and transposed (K-major for the GEMM)
    for tr in (False, True):
        s3 = torch.zeros_like(sd)
        q3 = torch.zeros((b, m, n) if tr else (b, n, m), dtype=torch.int8, device=gpu)
        ck.gemm_quantize_cols(b, n, m, xd.data_ptr(), s3.data_ptr(), q3.data_ptr(), tr, stream())
        assert_bits_equal(to_np(s3), s_ref, "gemm_quantize_cols scale (transposed=%s)" % tr)
        want = to_np(qd).transpose(0, 2, 1) if tr else to_np(qd)
        assert_bits_equal(to_np(q3), np.ascontiguousarray(want), "gemm_quantize_cols int8 (transposed=%s)" % tr)


def test_quantize_cols_more_teams_than_packet_slots(gpu):
    """4200 columns tiles x 2 parts exceed the 8192 packet slots of one launch: the batch goes out in several
    launches and must equal two half calls bit for bit; first and last entries against the oracle."""
    _name("quantize_cols, batch split over launches")
    b, n, m = 4200, 1000, 64
    gen = torch.Generator(device="cpu").manual_seed(6)
    x = (torch.randn(b, n, m, generator=gen) * 3).half().to(gpu)
    for tr in (False, True):
        sc = torch.zeros((b, m), dtype=torch.half, device=gpu); q = torch.zeros((b, m, n) if tr else (b, n, m), dtype=torch.int8, device=gpu)
        ck.gemm_quantize_cols(b, n, m, x.data_ptr(), sc.data_ptr(), q.data_ptr(), tr, stream())
        sc2 = torch.zeros_like(sc); q2 = torch.zeros_like(q)
        h = b // 2
        ck.gemm_quantize_cols(h, n, m, x.data_ptr(), sc2.data_ptr(), q2.data_ptr(), tr, stream())
        ck.gemm_quantize_cols(b - h, n, m, x[h:].data_ptr(), sc2[h:].data_ptr(), q2[h:].data_ptr(), tr, stream())
        assert_bits_equal(to_np(sc), to_np(sc2), "scales: one call == two half calls")
        assert_bits_equal(to_np(q), to_np(q2), "int8: one call == two half calls")
        for sl in (slice(0, 2), slice(b - 2, b), slice(4095, 4097)):
            xs = to_np(x[sl])
            s_ref = oracle.gemm_calc_scale_transpose(xs)
            q_ref = oracle.gemm_round_transpose(xs, s_ref)
            assert_bits_equal(to_np(sc[sl]), s_ref, "scales %s" % (sl,))
            assert_bits_equal(to_np(q[sl]), np.ascontiguousarray(q_ref.transpose(0, 2, 1)) if tr else q_ref, "int8 %s" % (sl,))


@pytest.mark.parametrize("rows0,rows1,m", [(512, 4096, 4096), (3, 0, 1000), (0, 7, 24), (5, 9, 30), (33, 17, 8200)])
def test_quantize_pair(gpu, rows0, rows1, m):
    """Two tensors with rows of one length quantised by one launch == each by itself."""
    _name("quantize_pair", rows0, rows1, m)
    rng = np.random.default_rng(rows0 * 31 + rows1 * 7 + m)
    xs = [adversarial_rows(rng, r, m) if r else np.zeros((0, m), np.float16) for r in (rows0, rows1)]
    d = [to_gpu(x) for x in xs]
    sc = [torch.empty((r,), dtype=torch.half, device=gpu) for r in (rows0, rows1)]
    q = [torch.empty((r, m), dtype=torch.int8, device=gpu) for r in (rows0, rows1)]
    ck.gemm_quantize_pair(rows0, d[0].data_ptr(), sc[0].data_ptr(), q[0].data_ptr(),
                          rows1, d[1].data_ptr(), sc[1].data_ptr(), q[1].data_ptr(), m, stream())
    for i, r in enumerate((rows0, rows1)):
        if r:
            s_ref = oracle.gemm_calc_scale(xs[i][None])
            assert_bits_equal(to_np(sc[i]), s_ref[0], "pair scale %d" % i)
            assert_bits_equal(to_np(q[i]), oracle.gemm_round(xs[i][None], s_ref)[0], "pair int8 %d" % i)


def test_quantisers_skip_nan_elements(gpu):
    """A NaN element (quiet or signalling) takes no part in a row's or a column's absmax -- the
    reference's fmaxf drops it (cuda/gemm.cu:68-72) -- and rounds to 0; the other elements of the
    row are quantised as if it were not there.  Rows with normal and with subnormal scales."""
    _name("quantisers with NaN elements")
    rng = np.random.default_rng(77)
    n, m = 40, 4096
    x = rand_half(rng, (1, n, m), 2.0)
    x[0, 5] *= np.float16(1e-4)                                   # subnormal scale
    bits_ = x.view(np.uint16)
    for r, c, pat in ((0, 0, 0x7e00), (3, 100, 0x7c01), (5, 7, 0xfe00), (9, 4095, 0xfdff), (9, 1, 0x7fff), (20, 2048, 0x7d55)):
        bits_[0, r, c] = pat
    xd = to_gpu(x)
    s_ref = oracle.gemm_calc_scale(x); q_ref = oracle.gemm_round(x, s_ref)
    assert np.isfinite(s_ref.astype(np.float32)).all()
    sd = torch.empty((1, n), dtype=torch.half, device=gpu); qd = torch.empty((1, n, m), dtype=torch.int8, device=gpu)
    ck.gemm_calc_scale(1, n, m, xd.data_ptr(), sd.data_ptr(), stream())
    assert_bits_equal(to_np(sd), s_ref, "calc_scale with NaN elements")
    sd.zero_()
    ck.gemm_quantize(1, n, m, xd.data_ptr(), sd.data_ptr(), qd.data_ptr(), False, stream())
    assert_bits_equal(to_np(sd), s_ref, "gemm_quantize scale with NaN elements")
    assert_bits_equal(to_np(qd), q_ref, "gemm_quantize int8 with NaN elements")
    assert to_np(qd)[0, 3, 100] == 0 and to_np(qd)[0, 9, 4095] == 0
    # columns: the same tensor transposed
    xt = np.ascontiguousarray(x.transpose(0, 2, 1)); xtd = to_gpu(xt)
    for tr in (False, True):
        sc = torch.zeros((1, n), dtype=torch.half, device=gpu)
        qc = torch.zeros((1, n, m) if tr else (1, m, n), dtype=torch.int8, device=gpu)
        ck.gemm_quantize_cols(1, m, n, xtd.data_ptr(), sc.data_ptr(), qc.data_ptr(), tr, stream())
        assert_bits_equal(to_np(sc), s_ref, "quantize_cols scale with NaN elements")
        assert_bits_equal(to_np(qc), q_ref if tr else np.ascontiguousarray(q_ref.transpose(0, 2, 1)), "quantize_cols int8 with NaN elements (transposed=%s)" % tr)


def test_round_unaligned_views(gpu):
    """Pointers that are only 2-byte aligned take the scalar kernels."""
    _name("round unaligned")
    rng = np.random.default_rng(5)
    x = rand_half(rng, (1, 6, 40))
    buf = torch.empty(x.size + 1, dtype=torch.half, device=gpu)
    buf[1:] = to_gpu(x).reshape(-1)
    sd = torch.empty((1, 6), dtype=torch.half, device=gpu)
    ck.gemm_calc_scale(1, 6, 40, buf.data_ptr() + 2, sd.data_ptr(), stream())
    assert_bits_equal(to_np(sd), oracle.gemm_calc_scale(x), "unaligned calc_scale")
    qd = torch.empty((1, 6, 40), dtype=torch.int8, device=gpu)
    ck.gemm_round(1, 6, 40, buf.data_ptr() + 2, sd.data_ptr(), qd.data_ptr(), stream())
    assert_bits_equal(to_np(qd), oracle.gemm_round(x, oracle.gemm_calc_scale(x)), "unaligned round")


def test_round_every_value_scale_pair(gpu):
    """gemm_round over ALL 65536 x 65536 (fp16 value, fp16 scale) pairs: the row kernels round
    through the row's reciprocal, which must equal divide-then-round everywhere.  The whole grid
    is checked on the device against gemm_round_transpose (per-element IEEE divide) on the
    transposed problem, and sampled scale rows against the oracle on the host."""
    _name("round all pairs")
    allh = torch.arange(65536, dtype=torch.int32, device=gpu).to(torch.int16).view(torch.half)   # every bit pattern
    x_row = allh.contiguous()
    rng = np.random.default_rng(11)
    CH = 4096                                           # scale patterns per chunk
    for c0 in range(0, 65536, CH):
        sc = allh[c0:c0 + CH].contiguous()              # (CH,)   row scales
        mat = x_row[None, :].expand(CH, 65536).contiguous()          # (CH, 65536): row i = all values
        out = torch.empty((CH, 65536), dtype=torch.int8, device=gpu)
        ck.gemm_round(1, CH, 65536, mat.data_ptr(), sc.data_ptr(), out.data_ptr(), stream())
        # same numbers with the roles of rows and columns swapped: element (j, i) = value j, scale i
        mat_t = x_row[:, None].expand(65536, CH).contiguous()
        out_t = torch.empty((65536, CH), dtype=torch.int8, device=gpu)
        ck.gemm_round_transpose(1, 65536, CH, mat_t.data_ptr(), sc.data_ptr(), out_t.data_ptr(), stream())
        assert torch.equal(out, out_t.t()), "reciprocal rounding differs from divide rounding, scales %d..%d" % (c0, c0 + CH)
        # the fused quantiser's rounding stage is the same code; pin sampled rows to the oracle
        rows = rng.integers(0, CH, 4)
        got = out[rows].cpu().numpy()
        xs = np.arange(65536, dtype=np.uint16).view(np.float16)
        for k, r in enumerate(rows):
            sr = np.array([[c0 + r]], dtype=np.uint16).view(np.float16)
            ref = oracle.gemm_round(xs[None, None, :], sr)
            assert_bits_equal(got[k], ref[0, 0], "oracle row, scale pattern %d" % (c0 + r))
        del mat, mat_t, out, out_t


@pytest.mark.parametrize("shape,bcx,bcy", [((1, 512, 4096), True, True), ((3, 20, 44), False, False),
                                          ((3, 20, 44), True, False), ((2, 7, 13), False, True),
                                          ((4, 128, 256), False, True)])
def test_gemm_scale(gpu, shape, bcx, bcy):
    _name("gemm_scale", shape, bcx, bcy)
    b, n, m = shape
    rng = np.random.default_rng(11 + n + m)
    acc = rng.integers(-2 ** 27, 2 ** 27, shape, dtype=np.int64).astype(np.int32)   # > 2^24: int->float rounds
    acc[0, 0, :4] = [0, 1, -1, 2 ** 31 - 1]
    sx = (rng.random((n if bcx else b * n,)) * 0.05 + 1e-4).astype(np.float16)
    sy = (rng.random((m if bcy else b * m,)) * 0.01 + 1e-5).astype(np.float16)
    accd, sxd, syd = to_gpu(acc), to_gpu(sx), to_gpu(sy)
    out = torch.empty(shape, dtype=torch.half, device=gpu)
    ck.gemm_scale(b, n, m, accd.data_ptr(), sxd.data_ptr(), syd.data_ptr(), out.data_ptr(), bcx, bcy, stream())
    assert_bits_equal(to_np(out), oracle.gemm_scale(acc, sx, sy, bcx, bcy), "gemm_scale")
    if not bcx:
        ck.gemm_scale_x(b, n, m, accd.data_ptr(), sxd.data_ptr(), out.data_ptr(), stream())
        assert_bits_equal(to_np(out), oracle.gemm_scale_x(acc, sx), "gemm_scale_x")
    if not bcy:
        ck.gemm_scale_y(b, n, m, accd.data_ptr(), syd.data_ptr(), out.data_ptr(), stream())
        assert_bits_equal(to_np(out), oracle.gemm_scale_y(acc, sy), "gemm_scale_y")


# ---------------------------------------------------------------------------------------------
# int8 GEMM: shapes of the reference's TEST_CASES (tests/test_gemm.py:43-60), every transpose
# combination, broadcast on either side; plus tile-boundary shapes.
# ---------------------------------------------------------------------------------------------
GEMM_CASES = [  # (batch, M, K, N) in the reference's bmm naming: kernel m = N, n = M
    (1, 4, 4, 4), (2, 4, 4, 4), (1, 8, 8, 8), (3, 12, 12, 12), (1, 16, 16, 16), (1, 32, 32, 32),
    (1, 64, 64, 64), (1, 128, 128, 128), (4, 128, 128, 128), (8, 112, 224, 112),
    (2, 512, 1024, 2048), (2, 500, 1024, 1996), (2, 512, 2560, 1024), (2, 1024, 512, 1024),
    (1, 260, 80, 132), (1, 256, 4096, 128), (1, 36, 16, 292),
]


def _gemm_case(gpu, m, k, n, bA, bB, aT, bT, rng, fused_too=True):
    A = rng.integers(-127, 128, (bA, m, k) if aT else (bA, k, m), dtype=np.int8)
    B = rng.integers(-127, 128, (bB, k, n) if bT else (bB, n, k), dtype=np.int8)
    if m * n * k * max(bA, bB) <= 2 ** 22:
        ref = oracle.gemm_int8(m, k, n, aT, bT, A, B)
    else:
        ref = oracle.gemm_int8_blas(m, k, n, aT, bT, A, B)
    batch = max(bA, bB)
    Ad, Bd = to_gpu(A), to_gpu(B)
    out = torch.full((batch, n, m), 12345, dtype=torch.int32, device=gpu)
    ck.gemm_int8(m, k, n, bA, bB, aT, bT, Ad.data_ptr(), Bd.data_ptr(), out.data_ptr(), stream())
    what = "gemm_int8 m=%d k=%d n=%d bA=%d bB=%d aT=%d bT=%d" % (m, k, n, bA, bB, aT, bT)
    assert_bits_equal(to_np(out), ref, what)
    if fused_too:
        bcr, bcc = bB == 1, bA == 1
        srow = (rng.random((n if bcr else batch * n,)) * 0.05 + 1e-4).astype(np.float16)
        scol = (rng.random((m if bcc else batch * m,)) * 0.01 + 1e-5).astype(np.float16)
        sr, sc = to_gpu(srow), to_gpu(scol)
        o16 = torch.empty((batch, n, m), dtype=torch.half, device=gpu)
        ck.gemm_int8_scale(m, k, n, bA, bB, aT, bT, Ad.data_ptr(), Bd.data_ptr(), sr.data_ptr(), sc.data_ptr(),
                           bcr, bcc, o16.data_ptr(), stream())
        assert_bits_equal(to_np(o16), oracle.gemm_scale(ref, srow, scol, bcr, bcc), what + " fused epilogue")


@pytest.mark.parametrize("case", GEMM_CASES)
def test_gemm_int8(gpu, case):
    batch, M, K, N = case
    rng = np.random.default_rng(M * 7919 + K * 31 + N)
    for aT in (False, True):
        for bT in (False, True):
            for (bA, bB) in {(batch, batch), (1, batch), (batch, 1)}:
                _name("gemm_int8", case, aT, bT, bA, bB)
                _gemm_case(gpu, N, K, M, bA, bB, aT, bT, rng)


# Tile-kernel coverage: K-major operands with k % 128 == 0 in every dispatch regime -- 256x256 tiles
# with a last round of half tiles, 128x128 and 128x64 tiles with the four-stage ring (one tile per
# workgroup, several with the next tile's slabs fetched ahead, slab counts that are not a multiple
# of the ring depth), ragged edges, output widths of 8j + 4 columns (fp16 rows that end in half a
# 16-byte piece and start on 8-byte boundaries: 8-byte stores; N = 7996 of the reference's
# tests/test_gemm.py:57 is such a width), one to many K slabs.
TILE_CASES = [  # (batch, kernel n = output rows, k, kernel m = output columns)
    (1, 4096, 512, 3072), (1, 2304, 256, 4608), (1, 2048, 1024, 2048), (1, 3000, 384, 2048), (2, 1500, 640, 1100),
    (1, 128, 128, 64), (1, 132, 128, 72), (1, 100, 256, 60), (3, 260, 384, 520), (1, 512, 128, 4096),
    (1, 520, 1152, 1032), (1, 1024, 896, 1028), (1, 640, 2048, 644), (4, 384, 512, 392), (1, 4100, 128, 2056),
    (1, 8, 128, 8), (1, 4, 256, 260), (2, 2816, 256, 2304), (1, 4096, 256, 3076), (2, 500, 1024, 1996), (1, 2052, 128, 4100),
    # depths of whole 64-byte but not whole 128-byte slabs: large and small tiles, one slab to many
    (1, 4096, 192, 3328), (1, 520, 448, 1032), (2, 132, 64, 72), (1, 2304, 1600, 2064), (3, 260, 320, 516),
    # depths of whole 16-byte pieces that are not whole slabs (the rest of the depth goes straight into the fragments):
    # one slab + 16 bytes, + 48 bytes, many slabs, large and small tiles, ragged edges
    (1, 132, 80, 72), (2, 260, 112, 516), (1, 4096, 208, 3328), (1, 2304, 1008, 2064), (3, 100, 144, 60), (1, 520, 4000, 1032),
    # ... and depths of whole dwords only (rows that start 4, 8 or 12 bytes into a 16-byte piece)
    (1, 520, 4100, 1032), (2, 260, 100, 516), (1, 4096, 212, 3328), (3, 132, 72, 72), (1, 300, 1000, 260),
]


@pytest.mark.parametrize("case", TILE_CASES)
def test_gemm_int8_tile_kernels(gpu, case):
    batch, n, k, m = case
    rng = np.random.default_rng(n * 7919 + k * 31 + m)
    for (bA, bB) in ((batch, batch),) + (((1, batch), (batch, 1)) if batch > 1 else ()):
        _name("gemm_int8 tile kernels", case, bA, bB)
        _gemm_case(gpu, m, k, n, bA, bB, True, False, rng)


# int8 operands with the contraction index as the row (the other three aT/bT combinations) on the tile kernel:
# k % 128 == 0 and row lengths that are multiples of 16; ragged tiles, one to several slabs, batch broadcast.
# (few 256 x 256 tiles: 128 x 128 tiles on the 32x32 form; enough of them for most compute units: the 16x16 form)
LAYOUT_CASES = [(1, 512, 256, 768), (2, 272, 128, 528), (1, 48, 384, 1040), (3, 1040, 640, 16), (1, 2304, 1024, 2064), (2, 2048, 256, 2560),
                (1, 4096, 256, 3088), (2, 3072, 128, 2064),
                # rows of a (K, rows) operand that are not whole 16-byte pieces (edge tiles that stay inside the matrix): small and large tiles
                (1, 500, 256, 1004), (3, 500, 128, 7996), (2, 132, 128, 260),
                # one operand stored (K, rows) and a depth beyond a slab that is not whole slabs (whole 16-byte pieces, whole dwords only)
                (1, 512, 200, 768), (2, 272, 500, 528), (1, 500, 132, 1004), (2, 132, 1000, 260)]


@pytest.mark.parametrize("case", LAYOUT_CASES)
def test_gemm_int8_tile_kernel_layouts(gpu, case):
    batch, n, k, m = case
    rng = np.random.default_rng(n * 7919 + k * 31 + m + 5)
    for aT, bT in ((True, True), (False, False), (False, True)):
        for (bA, bB) in ((batch, batch),) + (((1, batch), (batch, 1)) if batch > 1 else ()):
            _name("gemm_int8 tile kernel layouts", case, aT, bT, bA, bB)
            _gemm_case(gpu, m, k, n, bA, bB, aT, bT, rng)


def test_gemm_int8_extreme_values(gpu):
    """All operands -128 / 127: largest accumulators the int8 product can produce."""
    _name("gemm_int8 extremes")
    m, k, n = 256, 4096, 128
    for va, vb in ((-128, -128), (127, -128), (127, 127)):
        A = np.full((1, m, k), va, np.int8); B = np.full((1, n, k), vb, np.int8)
        out = torch.empty((1, n, m), dtype=torch.int32, device=gpu)
        Ad, Bd = to_gpu(A), to_gpu(B)
        ck.gemm_int8(m, k, n, 1, 1, True, False, Ad.data_ptr(), Bd.data_ptr(), out.data_ptr(), stream())
        assert (to_np(out) == va * vb * k).all()


def test_gemm_int8_config1_full(gpu):
    """The reference's own CPU-runnable case at full size (A [1,512,4096], W [1,4096,4096]) through the whole
    kernel-level pipeline, every stage bit-exact against the oracle."""
    _name("config1 full pipeline")
    g = torch.Generator().manual_seed(1001)
    A = torch.randn(1, 512, 4096, generator=g).half().numpy()
    W = (torch.randn(1, 4096, 4096, generator=g) * 0.02).half().numpy()
    sA, sW = oracle.gemm_calc_scale(A), oracle.gemm_calc_scale(W)
    qA, qW = oracle.gemm_round(A, sA), oracle.gemm_round(W, sW)
    acc = oracle.gemm_int8_blas(4096, 4096, 512, True, False, qW, qA)
    ref = oracle.gemm_scale(acc, sA, sW, True, True)
    Ad, Wd = to_gpu(A), to_gpu(W)
    sAd = torch.empty((1, 512), dtype=torch.half, device=gpu); sWd = torch.empty((1, 4096), dtype=torch.half, device=gpu)
    ck.gemm_calc_scale(1, 512, 4096, Ad.data_ptr(), sAd.data_ptr(), stream())
    ck.gemm_calc_scale(1, 4096, 4096, Wd.data_ptr(), sWd.data_ptr(), stream())
    qAd = torch.empty((1, 512, 4096), dtype=torch.int8, device=gpu); qWd = torch.empty((1, 4096, 4096), dtype=torch.int8, device=gpu)
    ck.gemm_round(1, 512, 4096, Ad.data_ptr(), sAd.data_ptr(), qAd.data_ptr(), stream())
    ck.gemm_round(1, 4096, 4096, Wd.data_ptr(), sWd.data_ptr(), qWd.data_ptr(), stream())
    assert_bits_equal(to_np(qAd), qA, "qA"); assert_bits_equal(to_np(qWd), qW, "qW")
    accd = torch.empty((1, 512, 4096), dtype=torch.int32, device=gpu)
    ck.gemm_int8(4096, 4096, 512, 1, 1, True, False, qWd.data_ptr(), qAd.data_ptr(), accd.data_ptr(), stream())
    assert_bits_equal(to_np(accd), acc, "int32 accumulators")
    outd = torch.empty((1, 512, 4096), dtype=torch.half, device=gpu)
    ck.gemm_scale(1, 512, 4096, accd.data_ptr(), sAd.data_ptr(), sWd.data_ptr(), outd.data_ptr(), True, True, stream())
    assert_bits_equal(to_np(outd), ref, "dequantised output")
    # loose check against the fp32 fake-quant formulation of the reference's test (tol 0.5 there)
    from oracle.formulations import quant_bmm_rowwise
    loose = quant_bmm_rowwise(torch.from_numpy(A), torch.from_numpy(W)).numpy()
    assert np.abs(to_np(outd).astype(np.float32) - loose).max() < 0.05


def test_gemm_int8_north_star_checksums(gpu):
    """M=4096, K=4096, N=10240 at full size: the int32 result must reproduce the exact row and
    column checksums  sum_i out[j,i] = P[j,:] . (sum_i Q[i,:])  and the transpose of that, which
    any wrong, missing or duplicated tile breaks; plus a random sample of entries."""
    _name("north-star checksums")
    M, K, N = 4096, 4096, 10240
    rng = np.random.default_rng(1000)
    qA = rng.integers(-127, 128, (1, M, K), dtype=np.int8)      # activations (rows of out)
    qW = rng.integers(-127, 128, (1, N, K), dtype=np.int8)      # weights (columns of out)
    out = torch.empty((1, M, N), dtype=torch.int32, device=gpu)
    qWd, qAd = to_gpu(qW), to_gpu(qA)
    ck.gemm_int8(N, K, M, 1, 1, True, False, qWd.data_ptr(), qAd.data_ptr(), out.data_ptr(), stream())
    o = to_np(out)[0].astype(np.int64)
    a64, w64 = qA[0].astype(np.int64), qW[0].astype(np.int64)
    assert np.array_equal(o.sum(axis=1), a64 @ w64.sum(axis=0))
    assert np.array_equal(o.sum(axis=0), w64 @ a64.sum(axis=0))
    jj = rng.integers(0, M, 2000); ii = rng.integers(0, N, 2000)
    assert np.array_equal(o[jj, ii], (a64[jj] * w64[ii]).sum(axis=1))


@pytest.mark.parametrize("M,K,N", [(2048, 512, 6144),      # 192 tiles of 256x256, one round, no half tiles
                                   (4096, 384, 4352),      # 272 tiles: 256 whole + 32 half tiles, three slabs (the ring position carries over)
                                   (2304, 128, 5888),      # 207 tiles of a single slab each
                                   (4100, 640, 4104),      # ragged edges in both directions
                                   # more 128x128 (128x64) tiles than compute units, at most two each: two workgroups share a
                                   # compute unit on a two-stage ring -- two slabs, one slab (fewer than stages), three
                                   (1536, 256, 4096), (1280, 128, 4096), (256, 384, 10240), (2048, 4096, 4096)])
def test_gemm_int8_large_tiles_exact(gpu, M, K, N):
    """Shapes that give every compute unit a 256x256 tile (the 16x16x64 MFMA form of the tile kernel) or two smaller
    ones at once: the int32 product checked exactly through row and column sums and 4000 sampled entries, the
    fused variant against gemm_scale of that product on the whole output."""
    _name("gemm large tiles", M, K, N)
    rng = np.random.default_rng(M + K + N)
    qA = rng.integers(-127, 128, (1, M, K), dtype=np.int8)
    qW = rng.integers(-127, 128, (1, N, K), dtype=np.int8)
    sA = (rng.random((1, M)) * 0.01 + 1e-3).astype(np.float16); sW = (rng.random((1, N)) * 0.01 + 1e-3).astype(np.float16)
    out = torch.empty((1, M, N), dtype=torch.int32, device=gpu)
    qWd, qAd, sAd, sWd = to_gpu(qW), to_gpu(qA), to_gpu(sA), to_gpu(sW)
    ck.gemm_int8(N, K, M, 1, 1, True, False, qWd.data_ptr(), qAd.data_ptr(), out.data_ptr(), stream())
    o = to_np(out)[0].astype(np.int64)
    a64, w64 = qA[0].astype(np.int64), qW[0].astype(np.int64)
    assert np.array_equal(o.sum(axis=1), a64 @ w64.sum(axis=0))
    assert np.array_equal(o.sum(axis=0), w64 @ a64.sum(axis=0))
    jj = rng.integers(0, M, 4000); ii = rng.integers(0, N, 4000)
    assert np.array_equal(o[jj, ii], (a64[jj] * w64[ii]).sum(axis=1))
    fused = torch.empty((1, M, N), dtype=torch.half, device=gpu)
    ck.gemm_int8_scale(N, K, M, 1, 1, True, False, qWd.data_ptr(), qAd.data_ptr(), sAd.data_ptr(), sWd.data_ptr(),
                       True, True, fused.data_ptr(), stream())
    two = torch.empty_like(fused)
    ck.gemm_scale(1, M, N, out.data_ptr(), sAd.data_ptr(), sWd.data_ptr(), two.data_ptr(), True, True, stream())
    assert torch.equal(two.view(torch.int16), fused.view(torch.int16)), "fused != gemm_int8 + gemm_scale"
    ref = oracle.gemm_scale(to_np(out)[:, :64], sA[:, :64], sW, True, True)
    assert_bits_equal(to_np(two)[:, :64], ref, "gemm_scale of the first 64 rows")


def test_north_star_fused_pipeline_bits(gpu):
    """The benchmarked call itself at full size -- quantise A [4096,4096] and W [10240,4096] (seed 1000, the
    bench's data), then the fused int8 GEMM + dequantisation -- checked to the bit on 64 output rows
    (four in every row tile, in both row halves of a tile) and all 10240 columns against the oracle's
    quantise -> exact integer product -> gemm_scale chain, and `ct.bmm` against the kernel-level calls
    on the whole output."""
    _name("north-star fused bits")
    import cpm_kernels_amd.torch as ct
    M, K, N = 4096, 4096, 10240
    g = torch.Generator().manual_seed(1000)
    A = torch.randn(1, M, K, generator=g).half()
    W = (torch.randn(1, N, K, generator=g) * 0.02).half()
    Ad, Wd = A.cuda(), W.cuda()
    sA = torch.empty((1, M), dtype=torch.half, device=gpu); qA = torch.empty((1, M, K), dtype=torch.int8, device=gpu)
    sW = torch.empty((1, N), dtype=torch.half, device=gpu); qW = torch.empty((1, N, K), dtype=torch.int8, device=gpu)
    ck.gemm_quantize(1, M, K, Ad.data_ptr(), sA.data_ptr(), qA.data_ptr(), False, stream())
    ck.gemm_quantize(1, N, K, Wd.data_ptr(), sW.data_ptr(), qW.data_ptr(), False, stream())
    out = torch.empty((1, M, N), dtype=torch.half, device=gpu)
    ck.gemm_int8_scale(N, K, M, 1, 1, True, False, qW.data_ptr(), qA.data_ptr(), sA.data_ptr(), sW.data_ptr(),
                       True, True, out.data_ptr(), stream())
    rows = np.array([t * 256 + off for t in range(16) for off in (3, 130, 200, 255)])
    An, Wn = A.numpy(), W.numpy()
    sWr = oracle.gemm_calc_scale(Wn); qWr = oracle.gemm_round(Wn, sWr)
    assert_bits_equal(to_np(sW), sWr, "W scales"); assert_bits_equal(to_np(qW), qWr, "W int8")
    Ar = np.ascontiguousarray(An[:, rows])
    sAr = oracle.gemm_calc_scale(Ar); qAr = oracle.gemm_round(Ar, sAr)
    assert_bits_equal(to_np(sA)[:, rows], sAr, "A scales (sampled rows)")
    assert_bits_equal(to_np(qA)[:, rows], qAr, "A int8 (sampled rows)")
    acc = oracle.gemm_int8_blas(N, K, len(rows), True, False, qWr, qAr)
    ref = oracle.gemm_scale(acc, sAr, sWr, True, True)
    assert_bits_equal(to_np(out)[:, rows], ref, "fused GEMM, sampled rows x all columns")
    # the int32 variant on the same operands, and the separate dequantisation of it
    acc_d = torch.empty((1, M, N), dtype=torch.int32, device=gpu)
    ck.gemm_int8(N, K, M, 1, 1, True, False, qW.data_ptr(), qA.data_ptr(), acc_d.data_ptr(), stream())
    assert_bits_equal(to_np(acc_d)[:, rows], acc, "int32 GEMM, sampled rows")
    two = torch.empty_like(out)
    ck.gemm_scale(1, M, N, acc_d.data_ptr(), sA.data_ptr(), sW.data_ptr(), two.data_ptr(), True, True, stream())
    assert torch.equal(two.view(torch.int16), out.view(torch.int16)), "fused != gemm_int8 + gemm_scale"
    del acc_d, two
    y = ct.bmm(Ad, False, Wd, True, int8=True)
    assert y.shape == (1, M, N) and torch.equal(y.view(torch.int16), out.view(torch.int16)), "ct.bmm != kernel-level calls"


# ---------------------------------------------------------------------------------------------
# decode GEMV
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("batch,dim_out,dim_in", [(32, 10240, 4096), (16, 4444, 8888), (1, 48, 256), (33, 100, 4096),
                                                  (130, 64, 512), (5, 17, 12), (128, 1000, 1040), (8, 40, 16),
                                                  # dim_in 4096 at 40, 36, 25 (odd) and 20 rows per workgroup, ragged ends; 16, 2 and 1 rows
                                                  (32, 10239, 4096), (17, 9000, 4096), (3, 6145, 4096), (16, 5000, 4096),
                                                  (7, 257, 4096), (1, 256, 4096), (31, 4096, 4096), (32, 10241, 4096),
                                                  # other row lengths of whole 256-byte chunks (the chunked kernel): the decode shapes of a 4096 / 10240 FFN
                                                  # and rows of 2048 and 8192 bytes, at one workgroup per compute unit with 16, 40 and ragged row counts
                                                  (32, 4096, 10240), (8, 4096, 10240), (1, 4096, 10240), (17, 4001, 10240), (32, 300, 10240),
                                                  (32, 4096, 8192), (5, 3333, 8192), (16, 100, 8192),
                                                  (32, 10240, 2048), (20, 7000, 2048), (3, 513, 2048), (32, 4096, 2048),
                                                  # and with more rows than one workgroup per compute unit holds
                                                  (32, 5000, 10240), (32, 12500, 2048),
                                                  # one to four vectors (the row-wise kernel): rows of 4 KB at 40, 40 ragged, 20, 17 and 12 rows per
                                                  # workgroup, rows of 10 KB at 16 rows (one and two vectors; three go to the chunked kernel)
                                                  (1, 10240, 4096), (2, 10240, 4096), (4, 10239, 4096), (1, 5000, 4096), (2, 4097, 4096), (4, 3000, 4096),
                                                  (3, 10240, 4096), (2, 4096, 10240), (1, 4001, 10240), (3, 4096, 10240)])
def test_gemv_broadcast_mat_int8(gpu, batch, dim_out, dim_in):
    _name("gemv", batch, dim_out, dim_in)
    rng = np.random.default_rng(1002 + dim_out)
    mat = rng.integers(-127, 128, (dim_out, dim_in), dtype=np.int8)
    vec = rng.integers(-127, 128, (batch, dim_in), dtype=np.int8)
    sm = (rng.random(dim_out) * 0.009 + 0.001).astype(np.float16)
    sv = (rng.random(batch) * 0.05 + 0.001).astype(np.float16)
    # exact reference: fp64 BLAS dot products are exact here, dequant via the oracle's gemm_scale
    acc = (vec.astype(np.float64) @ mat.astype(np.float64).T).astype(np.int32)[None]     # (1, batch, dim_out)
    ref = oracle.gemm_scale(acc, sv, sm, True, True)[0]
    if batch * dim_out * dim_in <= 2 ** 24:
        assert_bits_equal(oracle.gemv_broadcast_mat_int8(sm, mat, sv, vec), ref, "oracle gemv == gemm path")
    out = torch.empty((batch, dim_out), dtype=torch.half, device=gpu)
    md, vd, smd, svd = to_gpu(mat), to_gpu(vec), to_gpu(sm), to_gpu(sv)
    ck.gemv_broadcast_mat_int8(batch, dim_out, dim_in, smd.data_ptr(), md.data_ptr(), svd.data_ptr(), vd.data_ptr(),
                               out.data_ptr(), stream())
    assert_bits_equal(to_np(out), ref, "gemv_broadcast_mat_int8")
    # the invariant the reference tests (tests/test_gemv.py:49-59): GEMV == GEMM path
    if batch % 4 or dim_out % 4:
        return
    o2 = torch.empty((1, batch, dim_out), dtype=torch.half, device=gpu)
    ck.gemm_int8_scale(dim_out, dim_in, batch, 1, 1, True, False, md.data_ptr(), vd.data_ptr(), svd.data_ptr(),
                       smd.data_ptr(), True, True, o2.data_ptr(), stream())
    assert_bits_equal(to_np(o2)[0], to_np(out), "gemv == gemm_int8_scale")


# ---------------------------------------------------------------------------------------------
# layernorm / softmax / gelu (tolerance ops)
# ---------------------------------------------------------------------------------------------
LN_SHAPES = [(8, 4096, 512), (16, 768, 512), (4, 1024, 512), (3, 100, 40), (2, 33, 24), (2, 777, 123), (5, 4096, 1),
             (1, 5000, 64), (2, 2048, 32), (1, 1536, 8), (2, 64, 72), (2, 1100, 64), (1, 8192, 128), (1, 9000, 64),
             # widths that are not whole 16-byte pieces (8-byte, 4-byte, 2-byte accesses) on the tile and team kernels, and
             # widths whose rows do not start on cache-line boundaries (no non-temporal hint)
             (2, 4096, 500), (1, 3000, 77), (1, 4096, 38), (3, 640, 500), (2, 2048, 1000), (2, 900, 200)]


@pytest.mark.parametrize("shape", LN_SHAPES)
@pytest.mark.parametrize("rd_mean", [True, False])
def test_layernorm_forward(gpu, shape, rd_mean):
    _name("layernorm", shape, rd_mean)
    b, n, m = shape
    rng = np.random.default_rng(1003 + n + m)
    x = (rng.standard_normal(shape) * rng.uniform(0.5, 3.0) + (0.7 if rd_mean else 0.0)).astype(np.float16)
    for eps in (1e-5, 1e-3):
        ref = oracle.layernorm_forward(x, eps, rd_mean)
        xd = to_gpu(x)
        out = torch.empty_like(xd)
        ck.layernorm_forward(b, n, m, xd.data_ptr(), out.data_ptr(), eps, rd_mean, stream())
        # outputs are O(1); atol 2e-4 covers values next to zero where x - mean cancels
        assert_close_fp16(to_np(out), ref, rtol=1e-3, atol=2e-4, what="layernorm_forward %s" % (shape,))
        ck.layernorm_inplace_forward(b, n, m, xd.data_ptr(), eps, rd_mean, stream())
        # tall columns take a different kernel in place (another summation order), so the two
        # agree to the last fp16 bit only up to the rounding of the statistics
        assert_close_fp16(to_np(xd), ref, rtol=1e-3, atol=2e-4, what="layernorm_inplace_forward %s" % (shape,))
        assert_close_fp16(to_np(xd), to_np(out), rtol=1e-3, atol=2e-4, what="in place vs out of place")
    if m == 1:   # the reference pins step == forward(m=1) (tests/test_layernorm.py:115-152)
        xd = to_gpu(x); o2 = torch.empty_like(xd)
        ck.layernorm_step(b, n, xd.data_ptr(), o2.data_ptr(), 1e-3, rd_mean, stream())
        assert_bits_equal(to_np(o2), to_np(out), "layernorm_step == forward(m=1)")


def test_team_kernels_repeated_and_concurrent(gpu):
    """Tall columns are reduced by teams of workgroups that exchange partial results through a
    packet pool inside the library.  Back-to-back launches reuse the pool's regions, launches on
    two streams overlap in time, and in-place calls alias input and output: every result must
    equal the first one bit for bit (the team sums in part order, so results do not depend on
    timing) and match the oracle."""
    _name("team kernels")
    rng = np.random.default_rng(77)
    x = (rng.standard_normal((2, 3000, 192)) * 2 + 0.3).astype(np.float16)
    xs = (rng.standard_normal((2, 2500, 128)) * 4).astype(np.float16)
    xs[:, 1500:, :40] = -np.inf
    ln_ref = oracle.layernorm_forward(x, 1e-5, True)
    sm_ref = oracle.softmax_forward(xs)
    xd, xsd = to_gpu(x), to_gpu(xs)
    first_ln = torch.empty_like(xd); first_sm = torch.empty_like(xsd)
    ck.layernorm_forward(2, 3000, 192, xd.data_ptr(), first_ln.data_ptr(), 1e-5, True, stream())
    ck.softmax_forward(2, 2500, 128, xsd.data_ptr(), first_sm.data_ptr(), stream())
    assert_close_fp16(to_np(first_ln), ln_ref, rtol=1e-3, atol=2e-4, what="team layernorm")
    assert_close_fp16(to_np(first_sm), sm_ref, rtol=1e-3, atol=1e-7, what="team softmax")
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    outs = []
    torch.cuda.synchronize()
    for it in range(24):
        for s_ in (s1, s2):
            with torch.cuda.stream(s_):
                o1 = torch.empty_like(xd); o2 = xsd.clone()
                ck.layernorm_forward(2, 3000, 192, xd.data_ptr(), o1.data_ptr(), 1e-5, True, s_.cuda_stream)
                ck.softmax_inplace_forward(2, 2500, 128, o2.data_ptr(), s_.cuda_stream)
                outs.append((o1, o2))
    torch.cuda.synchronize()
    a, b = to_np(first_ln), to_np(first_sm)
    for k, (o1, o2) in enumerate(outs):
        assert_bits_equal(to_np(o1), a, "layernorm launch %d" % k)
        assert_bits_equal(to_np(o2), b, "softmax launch %d" % k)


def test_team_kernels_in_a_replayed_graph(gpu):
    """A captured launch is replayed with the same kernel arguments, packet pool region and tag
    included; each replay gets new input data and must give that data's result, not a mix with
    partial sums a previous replay left behind."""
    _name("team kernels, graph replay")
    rng = np.random.default_rng(78)
    shape_ln, shape_sm = (2, 2600, 128), (1, 4096, 192)
    xin = torch.empty(shape_ln, dtype=torch.half, device=gpu); xout = torch.empty_like(xin)
    sin = torch.empty(shape_sm, dtype=torch.half, device=gpu); sout = torch.empty_like(sin)

    def launches():
        ck.layernorm_forward(*shape_ln, xin.data_ptr(), xout.data_ptr(), 1e-5, True, stream())
        ck.softmax_forward(*shape_sm, sin.data_ptr(), sout.data_ptr(), stream())

    xin.normal_(); sin.normal_()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launches()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        launches()
    for it in range(5):
        x = (rng.standard_normal(shape_ln) * (1 + it) + it).astype(np.float16)
        sx = (rng.standard_normal(shape_sm) * 4).astype(np.float16)
        xin.copy_(to_gpu(x)); sin.copy_(to_gpu(sx))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        got_ln, got_sm = to_np(xout).copy(), to_np(sout).copy()
        launches()                                   # eager, same inputs
        assert_bits_equal(got_ln, to_np(xout), "layernorm replay %d == eager" % it)
        assert_bits_equal(got_sm, to_np(sout), "softmax replay %d == eager" % it)
        assert_close_fp16(got_ln, oracle.layernorm_forward(x, 1e-5, True), rtol=1e-3, atol=2e-4, what="replay %d layernorm" % it)
        assert_close_fp16(got_sm, oracle.softmax_forward(sx), rtol=1e-3, atol=1e-7, what="replay %d softmax" % it)


def test_team_kernels_more_teams_than_packet_slots(gpu):
    """3000 column tiles x 3 parts exceed the 8192 packet slots of one launch: layernorm and softmax then send
    the batch out in several launches.  One call must equal two half calls bit for bit, and the first, last and
    boundary batch entries must match the oracle."""
    _name("team kernels, batch split over launches")
    b, m = 3000, 64
    gen = torch.Generator(device=gpu).manual_seed(8)
    for name, n in (("layernorm", 1100), ("softmax", 2100)):
        x = torch.randn(b, n, m, generator=gen, device=gpu, dtype=torch.float32).mul_(3).half()
        y = torch.zeros_like(x); y2 = torch.zeros_like(x)
        h = b // 2

        def run(cnt, xin, out):
            if name == "layernorm":
                ck.layernorm_forward(cnt, n, m, xin.data_ptr(), out.data_ptr(), 1e-5, True, stream())
            else:
                ck.softmax_forward(cnt, n, m, xin.data_ptr(), out.data_ptr(), stream())
        run(b, x, y)
        run(h, x, y2)
        run(b - h, x[h:], y2[h:])
        assert_bits_equal(to_np(y), to_np(y2), name + ": one call == two half calls")
        per_launch = 8192 // 3
        for sl in (slice(0, 2), slice(b - 2, b), slice(per_launch - 1, per_launch + 1)):
            xs = to_np(x[sl])
            if name == "layernorm":
                assert_close_fp16(to_np(y[sl]), oracle.layernorm_forward(xs, 1e-5, True), rtol=1e-3, atol=2e-4, what="layernorm %s" % (sl,))
            else:
                assert_close_fp16(to_np(y[sl]), oracle.softmax_forward(xs), rtol=1e-3, atol=1e-7, max_ulp=2, what="softmax %s" % (sl,))
        del x, y, y2


def test_scheduled_softmax_in_a_replayed_graph(gpu):
    """The many-tile softmax hands out tiles from a counter in device memory that its last workgroup
    clears.  Replays of a captured graph (same counter slot every time), launches back to back and
    launches on two streams at once must each find a clean counter: every tile computed exactly once."""
    _name("scheduled softmax, graph replay")
    rng = np.random.default_rng(79)
    shape = (36, 1000, 1024)                      # 576 tiles: more than two per compute unit
    sin = torch.empty(shape, dtype=torch.half, device=gpu); sout = torch.empty_like(sin); sout2 = torch.empty_like(sin)

    def launches():
        ck.softmax_forward(*shape, sin.data_ptr(), sout.data_ptr(), stream())
        ck.softmax_forward(*shape, sin.data_ptr(), sout2.data_ptr(), stream())

    sin.normal_()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launches()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        launches()
    for it in range(4):
        sx = (rng.standard_normal(shape) * 4).astype(np.float16)
        sin.copy_(to_gpu(sx)); sout.zero_(); sout2.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        got, got2 = to_np(sout).copy(), to_np(sout2).copy()
        assert_bits_equal(got, got2, "two launches of one replay (%d)" % it)
        sout.zero_(); sout2.zero_()
        for _ in range(3):
            launches()                               # eager, back to back
        assert_bits_equal(got, to_np(sout), "replay %d == eager" % it)
        assert_bits_equal(got, to_np(sout2), "replay %d == eager (second output)" % it)
        if it == 0:
            assert_close_fp16(got, oracle.softmax_forward(sx), rtol=1e-3, atol=1e-7, max_ulp=2, what="scheduled softmax")
    # two streams at once
    other = torch.cuda.Stream()
    other.wait_stream(torch.cuda.current_stream())
    sout.zero_(); sout2.zero_()
    torch.cuda.synchronize()
    for _ in range(4):
        ck.softmax_forward(*shape, sin.data_ptr(), sout.data_ptr(), stream())
        with torch.cuda.stream(other):
            ck.softmax_forward(*shape, sin.data_ptr(), sout2.data_ptr(), other.cuda_stream)
    torch.cuda.synchronize()
    assert_bits_equal(to_np(sout), got, "stream A")
    assert_bits_equal(to_np(sout2), got, "stream B")


@pytest.mark.parametrize("shape", [(8, 4096, 512), (3, 100, 40), (2, 777, 124), (2, 1024, 64)])
@pytest.mark.parametrize("bias", [True, False])
def test_layernorm_affine_fused(gpu, shape, bias):
    """Fused norm+affine == layernorm_forward then arith_ln_mul_add / arith_ln_mul, bit for bit."""
    _name("layernorm affine", shape, bias)
    b, n, m = shape
    rng = np.random.default_rng(17 + n)
    x = rand_half(rng, shape)
    gamma = (1 + 0.1 * rng.standard_normal(n)).astype(np.float16)
    beta = (0.1 * rng.standard_normal(n)).astype(np.float16)
    xd, gd, bd = to_gpu(x), to_gpu(gamma), to_gpu(beta)
    two = torch.empty_like(xd)
    ck.layernorm_forward(b, n, m, xd.data_ptr(), two.data_ptr(), 1e-5, bias, stream())
    normed = to_np(two).copy()
    if bias:
        ck.arith_ln_mul_add(b, n, m, two.data_ptr(), gd.data_ptr(), bd.data_ptr(), two.data_ptr(), stream())
        assert_bits_equal(to_np(two), oracle.arith_ln_mul_add(normed, gamma, beta), "arith_ln_mul_add")
    else:
        ck.arith_ln_mul(b, n, m, two.data_ptr(), gd.data_ptr(), two.data_ptr(), stream())
        assert_bits_equal(to_np(two), oracle.arith_ln_mul(normed, gamma), "arith_ln_mul")
    one = torch.empty_like(xd)
    ck.layernorm_affine_forward(b, n, m, xd.data_ptr(), gd.data_ptr(), bd.data_ptr() if bias else None,
                                one.data_ptr(), 1e-5, bias, stream())
    assert_bits_equal(to_np(one), to_np(two), "fused == two launches")


SOFTMAX_SHAPES = [(1, 2, 32), (4, 128, 128), (4, 128, 16), (4, 123, 16), (16, 1024, 320), (7, 1024, 321),
                  (3, 512, 64), (2, 2000, 48), (2, 4096, 16), (1, 5000, 24), (6, 333, 1), (2, 64, 200), (2, 2100, 64),
                  (1, 4096, 192), (1, 8192, 64), (1, 9000, 64),
                  # several tiles per compute unit: the persistent kernel (ragged rows, ragged last column tile)
                  (40, 700, 1024), (64, 300, 520), (33, 1024, 1000), (600, 257, 64), (20, 1500, 1024), (70, 2048, 264),
                  # widths that are not whole 16-byte pieces on the tile and team kernels
                  (2, 2100, 500), (1, 3000, 77), (3, 1024, 1004), (2, 500, 38), (3, 1500, 250)]


@pytest.mark.parametrize("shape", SOFTMAX_SHAPES)
def test_softmax_forward(gpu, shape):
    _name("softmax", shape)
    b, n, m = shape
    rng = np.random.default_rng(1004 + n + m)
    x = rand_half(rng, shape, 4.0)
    if n >= 8 and m >= 4:
        x[0, : n // 2, 0] = -np.inf              # partially masked column
        x[0, :, 1] = -np.inf                     # fully masked column -> zeros, not NaN
        x[0, :, 2] = -np.inf; x[0, n // 3, 2] = 3.0     # one-hot -> exactly 1
        x[0, :, 3] = np.float16(2.5)             # constant -> 1/n
    ref = oracle.softmax_forward(x)
    xd = to_gpu(x); out = torch.empty_like(xd)
    ck.softmax_forward(b, n, m, xd.data_ptr(), out.data_ptr(), stream())
    got = to_np(out)
    # atol 1e-7: about two steps of the fp16 subnormal grid, where tiny probabilities live
    assert_close_fp16(got, ref, rtol=1e-3, atol=1e-7, max_ulp=2, what="softmax_forward %s" % (shape,))
    if n >= 8 and m >= 4:
        assert (got[0, :, 1] == 0).all()
        assert got[0, n // 3, 2] == 1.0 and got[0, :, 2].sum() == 1.0
    ck.softmax_inplace_forward(b, n, m, xd.data_ptr(), stream())
    assert_bits_equal(to_np(xd), got, "in place == out of place")
    if m == 1:   # tests/test_softmax.py:51-76 of the reference: step == forward(m=1)
        xs = to_gpu(x)
        ck.softmax_step_inplace(b, n, xs.data_ptr(), stream())
        assert_bits_equal(to_np(xs), got, "softmax_step_inplace == forward(m=1)")


def test_softmax_causal_full_size_properties(gpu):
    """Config 3 size, (64, 1024, 1024) slice count reduced to keep the CPU side in seconds:
    causal -inf above the diagonal; columns sum to 1, masked entries are exactly 0, and a
    sample of columns matches the oracle."""
    _name("softmax causal")
    b, n, m = 64, 1024, 1024
    g = torch.Generator().manual_seed(1003)
    s = (torch.randn(b, n, m, generator=g) * 4).half()
    kk = torch.arange(n)[:, None]; qq = torch.arange(m)[None, :]
    s.masked_fill_((kk > qq)[None], float("-inf"))
    xd = s.cuda(); out = torch.empty_like(xd)
    ck.softmax_forward(b, n, m, xd.data_ptr(), out.data_ptr(), stream())
    o = out.float()
    assert torch.all(o.masked_select((kk > qq)[None].cuda()) == 0)
    assert torch.allclose(o.sum(dim=1), torch.ones(b, m, device=gpu), atol=2e-3)
    ref = oracle.softmax_forward(s[:2].numpy())
    assert_close_fp16(to_np(out[:2]), ref, rtol=1e-3, atol=1e-7, max_ulp=2, what="softmax causal sample")


STEP_SHAPES = [(32, 4096), (32, 10240), (3, 4099), (128, 768), (1, 2), (7, 1024)]


@pytest.mark.parametrize("shape", STEP_SHAPES)
@pytest.mark.parametrize("rd_mean", [True, False])
def test_layernorm_step_decode_sizes(gpu, shape, rd_mean):
    """layernorm_step and layernorm_step_inplace at decode sizes: equal to forward(m=1) as the
    reference pins it (tests/test_layernorm.py:115-152, isclose 1e-5 there, bits here) and within
    1e-3 of the oracle."""
    _name("layernorm_step", shape, rd_mean)
    b, n = shape
    rng = np.random.default_rng(2003 + n)
    x = (rng.standard_normal(shape) * 1.7 + (0.4 if rd_mean else 0.0)).astype(np.float16)
    for eps in (1e-5, 1e-3):
        ref = oracle.layernorm_forward(x[:, :, None], eps, rd_mean)[:, :, 0]
        xd = to_gpu(x)
        fwd = torch.empty_like(xd); out = torch.empty_like(xd)
        ck.layernorm_forward(b, n, 1, xd.data_ptr(), fwd.data_ptr(), eps, rd_mean, stream())
        ck.layernorm_step(b, n, xd.data_ptr(), out.data_ptr(), eps, rd_mean, stream())
        assert_close_fp16(to_np(out), ref, rtol=1e-3, atol=2e-4, what="layernorm_step vs oracle")
        assert_bits_equal(to_np(out), to_np(fwd), "layernorm_step == forward(m=1)")
        ck.layernorm_step_inplace(b, n, xd.data_ptr(), eps, rd_mean, stream())
        assert_bits_equal(to_np(xd), to_np(out), "layernorm_step_inplace == layernorm_step")


@pytest.mark.parametrize("shape", STEP_SHAPES + [(3, 12321), (123, 321)])
def test_softmax_step_decode_sizes(gpu, shape):
    """softmax_step_inplace at decode sizes against forward(m=1) (tests/test_softmax.py:51-76 of the
    reference) and the oracle, with masked (-inf) entries and one fully masked row."""
    _name("softmax_step", shape)
    b, n = shape
    rng = np.random.default_rng(2004 + n)
    x = rand_half(rng, shape, 4.0)
    x[0, n // 2:] = -np.inf
    if b > 1:
        x[1, :] = -np.inf
    ref = oracle.softmax_forward(x[:, :, None])[:, :, 0]
    xd = to_gpu(x); fwd = torch.empty_like(xd)
    ck.softmax_forward(b, n, 1, xd.data_ptr(), fwd.data_ptr(), stream())
    ck.softmax_step_inplace(b, n, xd.data_ptr(), stream())
    assert_close_fp16(to_np(xd), ref, rtol=1e-3, atol=1e-7, max_ulp=2, what="softmax_step_inplace vs oracle")
    assert_bits_equal(to_np(xd), to_np(fwd), "softmax_step_inplace == forward(m=1)")
    assert (to_np(xd)[0, n // 2:] == 0).all()


def test_softmax_config3_full_size_properties(gpu):
    """The exact config-3 workload, [512,1024,1024] causal (the bench's tensor): masked entries exactly
    0, every column sums to 1, the first and last batch entries match the oracle, and the eight
    repeats of the 64 distinct score matrices give identical results."""
    _name("softmax config 3 full size")
    g = torch.Generator().manual_seed(1003)
    s = (torch.randn(64, 1024, 1024, generator=g) * 4).half()
    kk = torch.arange(1024)[:, None]; qq = torch.arange(1024)[None, :]
    s.masked_fill_((kk > qq)[None], float("-inf"))
    xd = s.cuda().repeat(8, 1, 1).contiguous()
    out = torch.empty_like(xd)
    ck.softmax_forward(512, 1024, 1024, xd.data_ptr(), out.data_ptr(), stream())
    torch.cuda.synchronize()
    masked = (kk > qq).cuda()
    for c in range(0, 512, 64):
        o = out[c:c + 64]
        assert torch.all(o.masked_select(masked[None]) == 0)
        assert torch.allclose(o.float().sum(dim=1), torch.ones(64, 1024, device=gpu), atol=2e-3)
        assert torch.equal(o.view(torch.int16), out[:64].view(torch.int16)), "repeat %d differs" % (c // 64)
    ref = oracle.softmax_forward(s[[0, 63]].numpy())
    assert_close_fp16(to_np(out[[448, 511]]), ref, rtol=1e-3, atol=1e-7, max_ulp=2, what="softmax config 3 sample")
    ck.softmax_inplace_forward(512, 1024, 1024, xd.data_ptr(), stream())
    assert torch.equal(xd.view(torch.int16), out.view(torch.int16)), "in place != out of place"


def test_gelu_all_fp16_inputs(gpu):
    _name("gelu exhaustive")
    x = np.arange(65536, dtype=np.uint16).view(np.float16).reshape(4, 16384)
    ref = oracle.gelu_forward(x)
    xd = to_gpu(x); out = torch.empty_like(xd)
    ck.gelu_forward(4, 16384, xd.data_ptr(), out.data_ptr(), stream())
    got = to_np(out)
    # Normal-range results: 1e-3 relative and at most one fp16 ulp from the restated reference.
    # Below the smallest normal fp16 (x < -4.1) the reference's own 1 + tanhf(u) has one or two
    # significant bits left (cuda/gelu.cu:14 adds 1 to a float within 1e-7 of -1), so its values
    # there are rounding noise around the true -|x| exp(-2|u|); the kernel evaluates
    # x / (1 + exp(-2u)), which does not cancel.  Both are within 4 steps of the subnormal grid.
    normal = np.abs(ref.astype(np.float64)) >= 6.2e-5
    fin = np.isfinite(ref)
    sel = normal | ~fin
    assert_close_fp16(np.where(sel, got, 0), np.where(sel, ref, 0), rtol=1e-3, atol=0.0, max_ulp=1, what="gelu_forward, normal range")
    assert_close_fp16(np.where(sel, 0, got), np.where(sel, 0, ref), rtol=0.0, atol=2.4e-7, what="gelu_forward, subnormal range")
    ck.gelu_inplace_forward(4, 16384, xd.data_ptr(), stream())
    assert_bits_equal(to_np(xd), got, "in place == out of place")
    # odd length / unaligned tail
    y = x.reshape(-1)[1000:1000 + 1237].copy().reshape(1, 1237)
    yd = to_gpu(y); o2 = torch.empty_like(yd)
    ck.gelu_forward(1, 1237, yd.data_ptr(), o2.data_ptr(), stream())
    assert_bits_equal(to_np(o2), got.reshape(-1)[1000:1000 + 1237].reshape(1, 1237), "gelu odd length")


# ---------------------------------------------------------------------------------------------
# position bias
# ---------------------------------------------------------------------------------------------
POS_CONFIGS = [(32, 12, 128, False), (32, 12, 128, True), (32, 24, 256, True), (128, 64, 128, True),
               (16, 64, 256, False), (16, 16, 512, True), (32, 64, 128, True)]


@pytest.mark.parametrize("cfg", POS_CONFIGS)
def test_position_embedding(gpu, cfg):
    _name("position", cfg)
    num_buckets, heads, max_distance, bidi = cfg
    table = torch.empty((max_distance,), dtype=torch.int32, device=gpu)
    ck.position_embedding_init(num_buckets, max_distance, table.data_ptr(), bidi, stream())
    t_ref = oracle.position_embedding_init(num_buckets, max_distance, bidi)
    assert_bits_equal(to_np(table), t_ref, "bucket table %s" % (cfg,))
    rng = np.random.default_rng(1005)
    w = rand_half(rng, (heads, num_buckets))
    wd = to_gpu(w)
    for (ql, kl) in ((128, 128), (77, 200), (1024, 16), (5, 3), (136, 50)):
        out = torch.empty((heads, kl, ql), dtype=torch.half, device=gpu)
        ck.position_embedding_forward(ql, kl, num_buckets, max_distance, heads, table.data_ptr(), wd.data_ptr(),
                                      out.data_ptr(), bidi, stream())
        ref = oracle.position_embedding_forward(ql, kl, num_buckets, max_distance, t_ref, w, bidi)
        assert_bits_equal(to_np(out), ref, "position_embedding_forward %s %d %d" % (cfg, ql, kl))
    o = torch.empty((heads, 300), dtype=torch.half, device=gpu)
    ck.position_embedding_step(150, 300, num_buckets, max_distance, heads, table.data_ptr(), wd.data_ptr(),
                               o.data_ptr(), bidi, stream())
    assert_bits_equal(to_np(o), oracle.position_embedding_step(150, 300, num_buckets, max_distance, t_ref, w, bidi),
                      "position_embedding_step")


def test_position_embedding_config5_size(gpu):
    """64 heads, 1024 x 1024, 32 buckets, max_distance 128, bidirectional: Toeplitz property at
    full size plus equality with the oracle."""
    _name("position config5")
    table = torch.empty((128,), dtype=torch.int32, device=gpu)
    ck.position_embedding_init(32, 128, table.data_ptr(), True, stream())
    g = torch.Generator().manual_seed(1005)
    w = (torch.randn(64, 32, generator=g) * 0.02).half()
    out = torch.empty((64, 1024, 1024), dtype=torch.half, device=gpu)
    wd = w.cuda()
    ck.position_embedding_forward(1024, 1024, 32, 128, 64, table.data_ptr(), wd.data_ptr(), out.data_ptr(), True,
                                  stream())
    torch.cuda.synchronize()
    assert torch.equal(out[:, 1:, 1:], out[:, :-1, :-1])          # depends on q - k only
    ref = oracle.position_embedding_forward(1024, 1024, 32, 128, oracle.position_embedding_init(32, 128, True),
                                            w.numpy(), True)
    assert_bits_equal(to_np(out), ref, "config 5 bias")


# ---------------------------------------------------------------------------------------------
# elementwise helpers
# ---------------------------------------------------------------------------------------------
# (rows that are not whole 16-byte pieces: pieces of eight that run over a row's end into the next channel; rows under eight)
@pytest.mark.parametrize("shape", [(8, 4096, 512), (3, 33, 10), (2, 5, 1232), (2, 7, 500), (1, 3, 6), (3, 4, 14)])
def test_elementwise(gpu, shape):
    _name("elementwise", shape)
    b, n, m = shape
    rng = np.random.default_rng(23 + m)
    x = rand_half(rng, shape, 30.0); y = rand_half(rng, shape, 0.01)
    alpha = rand_half(rng, (n,), 2.0); beta = rand_half(rng, (n,), 5.0)
    xd, yd, ad, bd = to_gpu(x), to_gpu(y), to_gpu(alpha), to_gpu(beta)
    out = torch.empty_like(xd)
    ck.arith_ln_mul_add(b, n, m, xd.data_ptr(), ad.data_ptr(), bd.data_ptr(), out.data_ptr(), stream())
    assert_bits_equal(to_np(out), oracle.arith_ln_mul_add(x, alpha, beta), "arith_ln_mul_add")
    ck.arith_ln_mul(b, n, m, xd.data_ptr(), ad.data_ptr(), out.data_ptr(), stream())
    assert_bits_equal(to_np(out), oracle.arith_ln_mul(x, alpha), "arith_ln_mul")
    ck.arith_element_add(b, n * m, xd.data_ptr(), yd.data_ptr(), out.data_ptr(), stream())
    assert_bits_equal(to_np(out), oracle.arith_element_add(x, y), "arith_element_add")
    msk = rng.random((b, m)) < 0.7
    md = to_gpu(msk)
    for value in (float("-inf"), 0.0, 1.5):
        ck.mask(b, n, m, xd.data_ptr(), md.data_ptr(), value, out.data_ptr(), stream())
        assert_bits_equal(to_np(out), oracle.mask(x, msk, value), "mask value=%r" % value)


# ---------------------------------------------------------------------------------------------
# fp16 products next to the path (fp32 accumulation; the bar is the 1e-3 of fp16 outputs)
# ---------------------------------------------------------------------------------------------
F16_GEMM_CASES = [  # (batch, n, k, m) in the kernel's convention: out (batch, n, m)
    (1, 4, 4, 4), (2, 6, 10, 8), (3, 34, 64, 20), (2, 256, 128, 260), (1, 512, 1024, 384), (2, 130, 192, 70),
    # shapes the MFMA tile kernel takes in every layout (k % 64 == 0, m % 8 == 0; n % 8 == 0 for a (k, n) operand):
    # few rows (64 x 256 tiles) and many, ragged edges, one and several slabs of K
    (2, 64, 128, 264), (3, 40, 192, 1032), (2, 60, 128, 264), (2, 264, 320, 520), (1, 136, 64, 256), (2, 24, 64, 8),
    # one slab of K and several 256 x 256 tiles per workgroup (attention scores): whole tiles only, and ragged edges
    (32, 512, 64, 768), (24, 520, 64, 776), (40, 520, 128, 264), (36, 300, 192, 520),
    # several slabs of K and enough 256 x 256 tiles for every compute unit (the 16x16 MFMA form of the tile kernel)
    (48, 512, 256, 512), (50, 520, 320, 264),
    # depths of whole 64-byte but not whole 128-byte slabs (96, 160, 224 halves): large and small tiles
    (32, 512, 96, 768), (2, 264, 160, 520), (3, 40, 224, 1032),
    # depths of whole 16-byte pieces (8 halves) that are not whole slabs: one slab + 8 halves, + 24, many slabs, large and small tiles
    (2, 264, 40, 520), (3, 40, 56, 1032), (32, 512, 72, 768), (2, 300, 1000, 260), (40, 520, 104, 264),
    # any even depth beyond a slab, also beside an operand stored (K, rows) (probabilities x values over 500 keys: few and many output rows)
    (4, 64, 500, 500), (2, 132, 200, 260), (3, 40, 100, 1004), (2, 264, 250, 520), (2, 48, 66, 264), (3, 300, 130, 136),
    # rows of a (K, rows) operand that are whole 8-byte but not whole 16-byte pieces (the reference's 500 x 7996 of tests/test_gemm.py:56):
    # edge tiles that stay inside the matrix, small and large tiles, and the 64 x 256 tiles of few output rows
    (2, 500, 128, 1004), (3, 500, 128, 7996), (2, 132, 64, 260), (4, 48, 192, 1004),
    # more 128 x 128 tiles than compute units, at most two each (two workgroups per compute unit, two-stage ring)
    (24, 512, 128, 512),
    # output rows of 8j + 4 halves on the tile kernels (8-byte stores): 128 x 128 tiles, and 256 x 256 on every compute unit
    (2, 520, 256, 1028), (40, 512, 256, 524)]


@pytest.mark.parametrize("case", F16_GEMM_CASES)
@pytest.mark.parametrize("aT", [False, True])
@pytest.mark.parametrize("bT", [False, True])
def test_gemm_fp16(gpu, case, aT, bT):
    _name("gemm_fp16", case, aT, bT)
    batch, n, k, m = case
    rng = np.random.default_rng(n * 7 + k * 3 + m + aT * 2 + bT)
    for bA, bB in ((batch, batch), (1, batch), (batch, 1)):
        A = rng.standard_normal((bA, m, k) if aT else (bA, k, m)).astype(np.float16)
        B = (rng.standard_normal((bB, k, n) if bT else (bB, n, k)) / np.sqrt(k)).astype(np.float16)
        Ad, Bd = to_gpu(A), to_gpu(B)
        out = torch.empty((batch, n, m), dtype=torch.half, device=gpu)
        ck.gemm_fp16(m, k, n, bA, bB, aT, bT, Ad.data_ptr(), Bd.data_ptr(), out.data_ptr(), stream())
        Aop = A.astype(np.float64) if aT else A.astype(np.float64).transpose(0, 2, 1)      # (bA, m, k)
        Bop = B.astype(np.float64).transpose(0, 2, 1) if bT else B.astype(np.float64)      # (bB, n, k)
        ref = np.einsum("bnk,bmk->bnm", np.broadcast_to(Bop, (batch, n, k)), np.broadcast_to(Aop, (batch, m, k)))
        # one fp16 rounding of an fp32-accumulated sum; atol covers sums that cancel to near zero
        assert_close_fp16(to_np(out), ref.astype(np.float16), rtol=1e-3, atol=1e-3, what="gemm_fp16 %s" % (case,))


@pytest.mark.parametrize("shape", [(4, 64, 256), (3, 33, 100), (2, 1000, 4096), (1, 7, 6),
                                   # short rows (lanes share a wave's rows) and rows of whole 256-byte chunks (matrix cores)
                                   (5, 70, 64), (2, 1000, 128), (3, 9, 8), (40, 300, 512), (33, 1100, 1024), (130, 48, 384),
                                   # short rows in numbers that put several loads in flight per lane (ragged ends, waves that
                                   # straddle two batch entries); a transposed product whose lanes leave the unrolled loop unevenly
                                   (301, 1021, 64), (140, 1000, 128), (520, 1024, 24), (64, 64, 1000),
                                   # rows of 128 halves and more that are not whole 256-byte chunks (the predicated matrix-core kernel for the
                                   # shared matrix): whole 16-byte pieces, whole dwords only, more than 32 vectors
                                   (5, 300, 200), (40, 1000, 2050), (3, 70, 130), (2, 600, 4544)])
def test_gemv_fp16_family(gpu, shape):
    _name("gemv fp16", shape)
    batch, dim_out, dim_in = shape
    rng = np.random.default_rng(dim_out + dim_in)
    vec = rng.standard_normal((batch, dim_in)).astype(np.float16)
    mat = (rng.standard_normal((batch, dim_out, dim_in)) / np.sqrt(dim_in)).astype(np.float16)
    vd, md = to_gpu(vec), to_gpu(mat)
    out = torch.empty((batch, dim_out), dtype=torch.half, device=gpu)
    ref = np.einsum("bok,bk->bo", mat.astype(np.float64), vec.astype(np.float64)).astype(np.float16)
    for fn in (ck.gemv_fp16, ck.gemv_fp16_light):
        out.zero_()
        fn(batch, dim_out, dim_in, md.data_ptr(), vd.data_ptr(), out.data_ptr(), stream())
        assert_close_fp16(to_np(out), ref, rtol=1e-3, atol=1e-3, what=fn.__name__)
    mt = to_gpu(np.ascontiguousarray(mat.transpose(0, 2, 1)))                # (batch, dim_in, dim_out)
    for fn in (ck.gemv_fp16_transpose, ck.gemv_fp16_transpose_light):
        out.zero_()
        fn(batch, dim_out, dim_in, mt.data_ptr(), vd.data_ptr(), out.data_ptr(), stream())
        assert_close_fp16(to_np(out), ref, rtol=1e-3, atol=1e-3, what=fn.__name__)
    m0 = to_gpu(mat[0])
    ref0 = np.einsum("ok,bk->bo", mat[0].astype(np.float64), vec.astype(np.float64)).astype(np.float16)
    for fn in (ck.gemv_broadcast_mat_fp16, ck.gemv_broadcast_mat_fp16_light):
        out.zero_()
        fn(batch, dim_out, dim_in, m0.data_ptr(), vd.data_ptr(), out.data_ptr(), stream())
        assert_close_fp16(to_np(out), ref0, rtol=1e-3, atol=1e-3, what=fn.__name__)


@pytest.mark.parametrize("shape", [(1, 10240, 4096), (2, 10240, 4096), (1, 4096, 4096), (2, 4096, 4096), (2, 5000, 4096),
                                   (1, 7777, 4096), (2, 2305, 4096), (1, 2304, 4096), (3, 10240, 4096),
                                   # rows of 10240 halves (the vectors shared through LDS)
                                   (1, 4096, 10240), (2, 4096, 10240), (1, 2305, 10240), (2, 7001, 10240), (1, 10240, 10240)])
def test_gemv_broadcast_mat_fp16_one_or_two_vectors(gpu, shape):
    """The decode shapes with one or two vectors (cuda/gemv.cu:137-164 serves them with the same kernel as any
    other batch): rows of 4096 or 10240 halves go to a kernel without matrix cores from 9 rows per compute unit on;
    ragged last shares, the smallest and largest share, and the neighbours that stay on the matrix cores."""
    _name("gemv broadcast fp16, few vectors", shape)
    batch, dim_out, dim_in = shape
    rng = np.random.default_rng(batch * 7 + dim_out)
    vec = rng.standard_normal((batch, dim_in)).astype(np.float16)
    mat = (rng.standard_normal((dim_out, dim_in)) / np.sqrt(dim_in)).astype(np.float16)
    vd, md = to_gpu(vec), to_gpu(mat)
    out = torch.full((batch, dim_out), float("nan"), dtype=torch.half, device=gpu)
    ck.gemv_broadcast_mat_fp16(batch, dim_out, dim_in, md.data_ptr(), vd.data_ptr(), out.data_ptr(), stream())
    ref = (vec.astype(np.float64) @ mat.astype(np.float64).T).astype(np.float16)
    assert_close_fp16(to_np(out), ref, rtol=1e-3, atol=1e-3, what="gemv_broadcast_mat_fp16 %s" % (shape,))
    # the same call again gives the same bits (fixed summation order)
    out2 = torch.empty_like(out)
    ck.gemv_broadcast_mat_fp16(batch, dim_out, dim_in, md.data_ptr(), vd.data_ptr(), out2.data_ptr(), stream())
    assert_bits_equal(to_np(out2), to_np(out), "repeat")


@pytest.mark.parametrize("shape", [(2, 64, 128), (3, 100, 77), (1, 4096, 33), (4, 24, 1)])
def test_embedding_and_kv_copy(gpu, shape):
    """Pure data movement next to the path: gathers from the embedding table and the copy of a
    decode step's hidden state into the key/value buffer (cuda/embedding.cu:6-37,90-103,
    cuda/utils.cu:13-29), against numpy indexing."""
    _name("embedding / copy_data_to_kv", shape)
    b, hidden, seq = shape
    rng = np.random.default_rng(hidden + seq)
    vocab = 211
    w = rand_half(rng, (vocab, hidden))
    ids = rng.integers(0, vocab, (b, seq)).astype(np.int32)
    wd, idd = to_gpu(w), to_gpu(ids)
    out = torch.empty((b, hidden, seq), dtype=torch.half, device=gpu)
    ck.embedding_forward(b, hidden, seq, idd.data_ptr(), wd.data_ptr(), out.data_ptr(), stream())
    assert_bits_equal(to_np(out), np.ascontiguousarray(w[ids].transpose(0, 2, 1)), "embedding_forward")
    step_ids = to_gpu(ids[:, 0].copy())
    o2 = torch.empty((b, hidden), dtype=torch.half, device=gpu)
    ck.embedding_step(b, hidden, step_ids.data_ptr(), wd.data_ptr(), o2.data_ptr(), stream())
    assert_bits_equal(to_np(o2), w[ids[:, 0]], "embedding_step")
    if hidden % 2 == 0:
        buf = rand_half(rng, (b, 9, hidden))
        bd = to_gpu(buf)
        ck.copy_data_to_kv(b, 9, hidden, o2.data_ptr(), bd.data_ptr(), 5, stream())
        want = buf.copy(); want[:, 5, :] = w[ids[:, 0]]
        assert_bits_equal(to_np(bd), want, "copy_data_to_kv")


def test_error_codes(gpu):
    """Bad arguments come back as RuntimeError from the C ABI / AssertionError from the asserts
    the reference has (kernels/gemm.py:139-140, gemv.py:65, arith.py:53,146)."""
    _name("errors")
    from cpm_kernels_amd.library import cpmk
    t = torch.zeros(64, dtype=torch.int8, device=gpu)
    with pytest.raises(AssertionError):
        ck.gemm_int8(6, 4, 4, 1, 1, False, False, t.data_ptr(), t.data_ptr(), t.data_ptr(), stream())
    with pytest.raises(AssertionError):
        ck.gemm_int8(4, 4, 4, 2, 3, False, False, t.data_ptr(), t.data_ptr(), t.data_ptr(), stream())
    with pytest.raises(AssertionError):
        ck.gemv_broadcast_mat_int8(1, 4, 6, 0, 0, 0, 0, 0, stream())
    with pytest.raises(RuntimeError, match="divisibility"):
        cpmk.gemm_int8(6, 4, 4, 1, 1, 0, 0, t.data_ptr(), t.data_ptr(), t.data_ptr(), None)
    with pytest.raises(RuntimeError, match="invalid argument"):
        cpmk.gemm_calc_scale(-1, 4, 4, t.data_ptr(), t.data_ptr(), None)
    # empty problems are no-ops
    ck.gemm_calc_scale(0, 4, 4, 0, 0, stream())
    ck.softmax_forward(2, 0, 4, 0, 0, stream())
    ck.gelu_forward(0, 16, 0, 0, stream())
