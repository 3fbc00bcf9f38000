"""GPU parity on seeded random shapes: the fixed lists of tests/test_parity_gpu.py name the sizes
each dispatch branch was written for; this sweep draws sizes around the boundaries those
branches switch on (tile edges, 16-byte pieces, slab counts, column heights of the register-
resident and team kernels) and runs the same checks, so a branch that is only right for the
sizes it was tuned on fails here.  Seeds are fixed: a failure names its case and reproduces.
"""
import numpy as np
import pytest

import test_parity_gpu as tp
import test_training_gpu as tt

pytestmark = pytest.mark.gpu


def _near(rng, anchors, spread, lo=1, step=1):
    """A size next to one of `anchors` (within +-spread), at least lo, a multiple of step."""
    v = int(rng.choice(anchors)) + int(rng.integers(-spread, spread + 1))
    v = max(lo, v)
    return max(step, (v // step) * step)


def _gemm_shapes(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        kind = int(rng.integers(0, 4))
        # every size is a multiple of 4, the reference's precondition (kernels/gemm.py:139-140)
        if kind == 0:       # anything else goes: the generic kernel and its guards
            m, k, n = (4 * int(rng.integers(1, 50)) for _ in range(3))
        elif kind == 1:     # K-major tile kernels: k % 128 == 0, ragged rows and columns
            k = 128 * int(rng.integers(1, 9))
            n = _near(rng, [64, 128, 256, 512, 768], 40, lo=4, step=4)
            m = _near(rng, [64, 128, 256, 512, 1024], 40, lo=4, step=int(rng.choice([4, 8])))
        elif kind == 2:     # depths that are not whole slabs: whole 16-byte pieces, or whole dwords only (under one slab: the
                            # register-staged kernel; beyond: the tile kernels, the rest of the depth straight into the fragments)
            k = int(rng.choice([16, 4])) * int(rng.integers(1, 40))
            n = _near(rng, [32, 128, 300], 30, lo=4, step=4)
            m = _near(rng, [32, 128, 300], 30, lo=4, step=4)
        else:               # stored (K, rows) layouts on the tile kernel: rows in whole 16-byte pieces
            k = 128 * int(rng.integers(1, 6))
            n = _near(rng, [48, 256, 528], 64, lo=16, step=16)
            m = _near(rng, [48, 256, 528], 64, lo=16, step=16)
        batch = int(rng.choice([1, 1, 2, 3]))
        out.append((batch, n, k, m))
    return out


@pytest.mark.parametrize("case", _gemm_shapes(20240, 64))
def test_random_gemm_int8(gpu, case):
    batch, n, k, m = case
    rng = np.random.default_rng(n * 7919 + k * 31 + m + batch)
    aT, bT = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    combos = [(batch, batch)] + ([(1, batch), (batch, 1)] if batch > 1 else [])
    for bA, bB in combos:
        for (x, y) in ((True, False), (aT, bT)):       # the K-major fast path and one drawn layout
            tp._name("random gemm_int8", case, x, y, bA, bB)
            tp._gemm_case(gpu, m, k, n, bA, bB, x, y, rng)


def _quant_shapes(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        b = int(rng.choice([1, 1, 2, 3]))
        n = _near(rng, [8, 64, 256, 512, 1024, 2048, 2500], 24, lo=1)
        m = _near(rng, [8, 64, 128, 512, 1000, 4096], 40, lo=1, step=int(rng.choice([1, 2, 8])))
        if b * n * m > 6_000_000:
            m = max(8, 6_000_000 // (b * n) // 8 * 8)
        out.append((b, n, m))
    return out


@pytest.mark.parametrize("shape", _quant_shapes(20241, 40))
def test_random_quantisers(gpu, shape):
    tp.test_calc_scale_and_round(gpu, shape)
    tp.test_calc_scale_and_round_transpose(gpu, shape)


def _dim1_shapes(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        b = int(rng.choice([1, 2, 3, 5]))
        n = _near(rng, [1, 64, 256, 512, 1024, 2048, 4096, 5000], 20, lo=1)
        m = _near(rng, [1, 8, 64, 72, 128, 520], 12, lo=1, step=int(rng.choice([1, 8])))
        if b * n * m > 5_000_000:
            b = 1
        out.append((b, n, m))
    return out


@pytest.mark.parametrize("shape", _dim1_shapes(20242, 56))
def test_random_layernorm_softmax(gpu, shape):
    tp.test_layernorm_forward(gpu, shape, True)
    tp.test_layernorm_forward(gpu, shape, False)
    tp.test_softmax_forward(gpu, shape)


def _gemv_shapes(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        batch = int(rng.choice([1, 2, 7, 16, 32, 33, 40]))
        dim_out = _near(rng, [4, 100, 1024, 4096, 10240], 50, lo=1)
        dim_in = _near(rng, [4, 256, 1024, 4096], 64, lo=4, step=int(rng.choice([4, 16, 256])))
        out.append((batch, dim_out, dim_in))
    return out


@pytest.mark.parametrize("shape", _gemv_shapes(20243, 40))
def test_random_gemv_int8(gpu, shape):
    tp.test_gemv_broadcast_mat_int8(gpu, *shape)


def _f16_gemm_shapes(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        kind = int(rng.integers(0, 4))
        if kind == 0:       # even sizes only (kernels/gemm.py:200): the generic kernel
            n, k, m = (2 * int(rng.integers(1, 80)) for _ in range(3))
        elif kind == 3:     # any even depth beyond a slab on the tile kernels (the rest of the depth straight into the fragments),
                            # output rows of whole 8-byte pieces
            k = 2 * int(rng.integers(17, 300))
            n = _near(rng, [24, 64, 136, 264, 520], 24, lo=8, step=int(rng.choice([4, 8])))
            m = _near(rng, [64, 256, 520], 24, lo=8, step=int(rng.choice([4, 8])))
        elif kind == 1:     # tile kernel: k % 64 == 0, output rows of whole 16-byte pieces
            k = 64 * int(rng.integers(1, 8))
            n = _near(rng, [24, 64, 136, 264, 520], 24, lo=8, step=8)
            m = _near(rng, [64, 256, 520, 1032], 24, lo=8, step=8)
        else:               # same with ragged rows (a (k, n) operand then takes the generic kernel)
            k = 64 * int(rng.integers(1, 5))
            n = _near(rng, [30, 130, 270], 20, lo=2, step=2)
            m = _near(rng, [64, 256, 520], 24, lo=8, step=8)
        out.append((int(rng.choice([1, 2, 3])), n, k, m))
    return out


@pytest.mark.parametrize("case", _f16_gemm_shapes(20244, 32))
def test_random_gemm_fp16(gpu, case):
    rng = np.random.default_rng(sum(case))
    tp.test_gemm_fp16(gpu, case, True, False)
    tp.test_gemm_fp16(gpu, case, bool(rng.integers(0, 2)), True)


def _gemv_f16_shapes(seed, count):
    rng = np.random.default_rng(seed)
    return [(int(rng.choice([1, 3, 32, 40, 130])), _near(rng, [8, 64, 300, 1024], 40, lo=1),
             _near(rng, [8, 64, 128, 384, 1024, 4096], 32, lo=2, step=int(rng.choice([2, 8, 128]))))
            for _ in range(count)]


@pytest.mark.parametrize("shape", _gemv_f16_shapes(20245, 32))
def test_random_gemv_fp16(gpu, shape):
    tp.test_gemv_fp16_family(gpu, shape)


def _col_shapes(seed, count):
    """(batch, n, m) for the dim-1 reductions of the training kernels: column heights around the
    register-resident limit and the team sizes, widths with and without 16-byte accesses."""
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        b = int(rng.choice([1, 2, 3, 9]))
        n = _near(rng, [2, 64, 512, 1024, 2048, 4096, 6000], 24, lo=1)
        m = _near(rng, [2, 8, 64, 128, 200, 520], 10, lo=2, step=int(rng.choice([2, 8])))
        if b * n * m > 4_000_000:
            b = 1
        out.append((b, n, m))
    return out


@pytest.mark.parametrize("shape", _col_shapes(20246, 40))
def test_random_training_reductions(gpu, shape):
    tt.test_softmax_backward(gpu, shape)
    tt.test_layernorm_training_kernels(gpu, shape)
    tt.test_gemm_backward_quantisers(gpu, shape, bool(sum(shape) % 2))


@pytest.mark.parametrize("shape", [(int(b), int(n), int(m)) for b, n, m in
                                   np.random.default_rng(20247).integers(1, 300, (24, 3))])
def test_random_transposes(gpu, shape):
    tt.test_transpose(gpu, shape)
    tt.test_transpose_i8(gpu, shape)


def _bmm_shapes(seed, count):
    """(batch, M, K, N) of the torch-level bmm: multiples of 4, around the tile kernels' K % 128 and
    16-byte conditions (the column quantisers and int8 transposes switch kernels on the same sizes)."""
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        K = int(rng.choice([4 * int(rng.integers(1, 40)), 16 * int(rng.integers(1, 30)), 128 * int(rng.integers(1, 6))]))
        M = _near(rng, [8, 64, 136, 264, 520], 20, lo=4, step=int(rng.choice([4, 16])))
        N = _near(rng, [8, 64, 136, 264, 520], 20, lo=4, step=int(rng.choice([4, 16])))
        out.append((int(rng.choice([1, 2, 3])), M, K, N))
    return out


@pytest.mark.parametrize("case", _bmm_shapes(20248, 24))
def test_random_bmm_forward_backward(gpu, case):
    import test_torch_gpu as tg
    import test_torch_backward_gpu as tb
    rng = np.random.default_rng(sum(case))
    aT, bT = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    tg.test_bmm_int8(gpu, case, aT, bT)
    tb.test_bmm_backward(gpu, case, aT, bT, "int8")
    tb.test_bmm_backward(gpu, case, not aT, bT, "fp16")
