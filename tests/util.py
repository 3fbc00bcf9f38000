"""Helpers shared by the parity tests."""
import numpy as np
import torch


def stream():
    return torch.cuda.current_stream().cuda_stream


def to_gpu(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def to_np(t: torch.Tensor) -> np.ndarray:
    torch.cuda.synchronize()
    return t.detach().cpu().numpy()


def bits(a: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(a).view(np.uint16 if a.dtype == np.float16 else a.dtype)


def assert_bits_equal(actual: np.ndarray, expected: np.ndarray, what=""):
    a, e = bits(actual), bits(expected)
    assert a.shape == e.shape, (what, a.shape, e.shape)
    if not np.array_equal(a, e):
        bad = np.flatnonzero(a.ravel() != e.ravel())
        i = bad[0]
        raise AssertionError("%s: %d of %d elements differ; first at flat index %d: got %r expected %r" % (
            what, bad.size, a.size, i, actual.ravel()[i], expected.ravel()[i]))


def ordinal16(h: np.ndarray) -> np.ndarray:
    """Map fp16 bit patterns to integers that are monotone in the value (for ulp distances)."""
    u = bits(h).astype(np.int32)
    return np.where(u & 0x8000, -(u & 0x7fff), u)


def assert_close_fp16(actual, expected, rtol=1e-3, atol=0.0, max_ulp=None, what=""):
    """|a - e| <= rtol*|e| + atol elementwise (the 1e-3 relative bar of the path's fp16 outputs),
    optionally also a bound in fp16 ulps.  NaN/inf must match exactly."""
    a = np.asarray(actual); e = np.asarray(expected)
    assert a.shape == e.shape, (what, a.shape, e.shape)
    af, ef = a.astype(np.float64), e.astype(np.float64)
    fin = np.isfinite(ef)
    assert np.array_equal(np.isnan(af), np.isnan(ef)), what + ": NaN pattern differs"
    assert np.array_equal(af[~fin & ~np.isnan(ef)], ef[~fin & ~np.isnan(ef)]), what + ": inf differs"
    err = np.abs(af[fin] - ef[fin]); tol = rtol * np.abs(ef[fin]) + atol
    if not (err <= tol).all():
        i = int(np.argmax(err - tol))
        raise AssertionError("%s: %d of %d outside tolerance; worst got %r expected %r" % (
            what, int((err > tol).sum()), err.size, af[fin][i], ef[fin][i]))
    if max_ulp is not None:
        d = np.abs(ordinal16(a.astype(np.float16)) - ordinal16(e.astype(np.float16)))[fin]
        assert d.max(initial=0) <= max_ulp, "%s: max fp16 ulp distance %d > %d" % (what, d.max(), max_ulp)


def rand_half(rng, shape, std=1.0):
    return (rng.standard_normal(shape) * std).astype(np.float16)
