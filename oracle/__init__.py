"""CPU oracle for the int8 quantized-GEMM inference path -- TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import this package; nothing under ``cpm_kernels_amd/`` does.  It wraps ``cpmk_oracle.c`` (a
scalar C restatement of the reference's CUDA kernels, each function citing the reference
file:line it follows) behind numpy arrays, and adds an exact BLAS-backed int8 product for
sizes the scalar loops cannot finish in seconds.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libcpmk_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile cpmk_oracle.c with gcc (``make -C oracle``)."""
    if force or not os.path.exists(_LIB_PATH) or \
            os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "cpmk_oracle.c")):
        args = ["make", "-C", _HERE] + (["-B"] if force else [])
        subprocess.run(args, check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(build())
    return _lib


def _p(a: np.ndarray):
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(ctypes.c_void_p)


def _h(a) -> np.ndarray:
    a = np.ascontiguousarray(a)
    assert a.dtype == np.float16, a.dtype
    return a


I32, I64, F32 = ctypes.c_int32, ctypes.c_int64, ctypes.c_float


# ---- conversions (exported so the tests can pin them) ---------------------------------------
def half_to_float(h: np.ndarray) -> np.ndarray:
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().o_half_to_float(I64(h.size), _p(h), _p(out))
    return out


def float_to_half(f: np.ndarray) -> np.ndarray:
    f = np.ascontiguousarray(f, dtype=np.float32)
    out = np.empty(f.shape, np.uint16)
    lib().o_float_to_half(I64(f.size), _p(f), _p(out))
    return out


def double_to_half(d: np.ndarray) -> np.ndarray:
    d = np.ascontiguousarray(d, dtype=np.float64)
    out = np.empty(d.shape, np.uint16)
    lib().o_double_to_half(I64(d.size), _p(d), _p(out))
    return out


# ---- quantisation ---------------------------------------------------------------------------
def gemm_calc_scale(mat):
    mat = _h(mat); b, n, m = mat.shape
    out = np.empty((b, n), np.float16)
    lib().o_gemm_calc_scale(I32(b), I32(n), I32(m), _p(mat), _p(out))
    return out


def gemm_calc_scale_transpose(mat):
    mat = _h(mat); b, n, m = mat.shape
    out = np.empty((b, m), np.float16)
    lib().o_gemm_calc_scale_transpose(I32(b), I32(n), I32(m), _p(mat), _p(out))
    return out


def gemm_round(mat, scale):
    mat = _h(mat); scale = _h(scale); b, n, m = mat.shape
    assert scale.shape == (b, n)
    out = np.empty((b, n, m), np.int8)
    lib().o_gemm_round(I32(b), I32(n), I32(m), _p(mat), _p(scale), _p(out))
    return out


def gemm_round_transpose(mat, scale):
    mat = _h(mat); scale = _h(scale); b, n, m = mat.shape
    assert scale.shape == (b, m)
    out = np.empty((b, n, m), np.int8)
    lib().o_gemm_round_transpose(I32(b), I32(n), I32(m), _p(mat), _p(scale), _p(out))
    return out


def gemm_scale(acc, scale_x, scale_y, broad_cast_x, broad_cast_y):
    acc = np.ascontiguousarray(acc, dtype=np.int32); b, n, m = acc.shape
    scale_x = _h(scale_x); scale_y = _h(scale_y)
    assert scale_x.size == (n if broad_cast_x else b * n) and scale_y.size == (m if broad_cast_y else b * m)
    out = np.empty((b, n, m), np.float16)
    lib().o_gemm_scale(I32(b), I32(n), I32(m), _p(acc), _p(scale_x), _p(scale_y), _p(out),
                       ctypes.c_int(int(broad_cast_x)), ctypes.c_int(int(broad_cast_y)))
    return out


def gemm_scale_x(acc, scale_x):
    acc = np.ascontiguousarray(acc, dtype=np.int32); b, n, m = acc.shape
    out = np.empty((b, n, m), np.float16)
    lib().o_gemm_scale_x(I32(b), I32(n), I32(m), _p(acc), _p(_h(scale_x)), _p(out))
    return out


def gemm_scale_y(acc, scale_y):
    acc = np.ascontiguousarray(acc, dtype=np.int32); b, n, m = acc.shape
    out = np.empty((b, n, m), np.float16)
    lib().o_gemm_scale_y(I32(b), I32(n), I32(m), _p(acc), _p(_h(scale_y)), _p(out))
    return out


# ---- int8 GEMM ------------------------------------------------------------------------------
def _check_gemm(m, k, n, aT, bT, A, B):
    A = np.ascontiguousarray(A, dtype=np.int8); B = np.ascontiguousarray(B, dtype=np.int8)
    assert A.ndim == 3 and B.ndim == 3
    assert A.shape[1:] == ((m, k) if aT else (k, m)), (A.shape, m, k, aT)
    assert B.shape[1:] == ((k, n) if bT else (n, k)), (B.shape, n, k, bT)
    bA, bB = A.shape[0], B.shape[0]
    assert bA == bB or bA == 1 or bB == 1
    return A, B, bA, bB


def gemm_int8(m, k, n, aT, bT, A, B):
    """Scalar loops (cpmk_oracle.c:o_gemm_int8); use for small shapes."""
    A, B, bA, bB = _check_gemm(m, k, n, aT, bT, A, B)
    out = np.empty((max(bA, bB), n, m), np.int32)
    lib().o_gemm_int8(I32(m), I32(k), I32(n), I32(bA), I32(bB), ctypes.c_int(int(aT)), ctypes.c_int(int(bT)),
                      _p(A), _p(B), _p(out))
    return out


def gemm_int8_blas(m, k, n, aT, bT, A, B):
    """Same product through float32 BLAS on k-chunks of 1024: every partial sum is an integer
    below 1024 * 128^2 = 2^24, so fp32 accumulation is exact, and the chunks are added in
    int64.  Pinned against the scalar loops by tests/test_oracle.py."""
    A, B, bA, bB = _check_gemm(m, k, n, aT, bT, A, B)
    batch = max(bA, bB)
    out = np.zeros((batch, n, m), np.int64)
    for b in range(batch):
        a = A[0 if bA == 1 else b]; bb = B[0 if bB == 1 else b]
        a_km = a.T if aT else a            # (k, m)
        b_nk = bb.T if bT else bb          # (n, k)
        for k0 in range(0, k, 1024):
            pa = np.ascontiguousarray(a_km[k0:k0 + 1024], dtype=np.float32)
            pb = np.ascontiguousarray(b_nk[:, k0:k0 + 1024], dtype=np.float32)
            out[b] += (pb @ pa).astype(np.int64)
    assert np.abs(out).max(initial=0) < 2 ** 31
    return out.astype(np.int32)


# ---- GEMV -----------------------------------------------------------------------------------
def gemv_calc_scale(vec):
    vec = _h(vec); b, n = vec.shape
    out = np.empty((b,), np.float16)
    lib().o_gemv_calc_scale(I32(b), I32(n), _p(vec), _p(out))
    return out


def gemv_round(vec, scale):
    vec = _h(vec); scale = _h(scale); b, n = vec.shape
    out = np.empty((b, n), np.int8)
    lib().o_gemv_round(I32(b), I32(n), _p(vec), _p(scale), _p(out))
    return out


def gemv_broadcast_mat_int8(scale_mat, mat, scale_vec, vec):
    mat = np.ascontiguousarray(mat, dtype=np.int8); vec = np.ascontiguousarray(vec, dtype=np.int8)
    dim_out, dim_in = mat.shape; batch = vec.shape[0]
    assert vec.shape[1] == dim_in
    out = np.empty((batch, dim_out), np.float16)
    lib().o_gemv_broadcast_mat_int8(I32(batch), I32(dim_out), I32(dim_in), _p(_h(scale_mat)), _p(mat),
                                    _p(_h(scale_vec)), _p(vec), _p(out))
    return out


# ---- normalisation, softmax, gelu -----------------------------------------------------------
def layernorm_forward(mat, eps, rd_mean):
    mat = _h(mat); b, n, m = mat.shape
    out = np.empty_like(mat)
    lib().o_layernorm_forward(I32(b), I32(n), I32(m), _p(mat), _p(out), F32(eps), ctypes.c_int(int(rd_mean)))
    return out


def softmax_forward(x):
    x = _h(x); b, n, m = x.shape
    out = np.empty_like(x)
    lib().o_softmax_forward(I32(b), I32(n), I32(m), _p(x), _p(out))
    return out


def gelu_forward(x):
    x = _h(x)
    out = np.empty_like(x)
    lib().o_gelu_forward(I64(x.size), _p(x), _p(out))
    return out


# ---- position bias --------------------------------------------------------------------------
def position_embedding_init(num_buckets, max_distance, bidirectional):
    out = np.empty((max_distance,), np.int32)
    lib().o_position_embedding_init(I32(num_buckets), I32(max_distance), _p(out), ctypes.c_int(int(bidirectional)))
    return out


def position_embedding_forward(query_len, key_len, num_buckets, max_distance, mapping, weight, bidirectional):
    weight = _h(weight); heads = weight.shape[0]
    mapping = np.ascontiguousarray(mapping, dtype=np.int32)
    out = np.empty((heads, key_len, query_len), np.float16)
    lib().o_position_embedding_forward(I32(query_len), I32(key_len), I32(num_buckets), I32(max_distance), I32(heads),
                                       _p(mapping), _p(weight), _p(out), ctypes.c_int(int(bidirectional)))
    return out


def position_embedding_step(query_pos, key_len, num_buckets, max_distance, mapping, weight, bidirectional):
    weight = _h(weight); heads = weight.shape[0]
    mapping = np.ascontiguousarray(mapping, dtype=np.int32)
    out = np.empty((heads, key_len), np.float16)
    lib().o_position_embedding_step(I32(query_pos), I32(key_len), I32(num_buckets), I32(max_distance), I32(heads),
                                    _p(mapping), _p(weight), _p(out), ctypes.c_int(int(bidirectional)))
    return out


# ---- elementwise ----------------------------------------------------------------------------
def arith_ln_mul_add(x, alpha, beta):
    x = _h(x); b, n, m = x.shape
    out = np.empty_like(x)
    lib().o_arith_ln_mul_add(I32(b), I32(n), I32(m), _p(x), _p(_h(alpha)), _p(_h(beta)), _p(out))
    return out


def arith_ln_mul(x, alpha):
    x = _h(x); b, n, m = x.shape
    out = np.empty_like(x)
    lib().o_arith_ln_mul(I32(b), I32(n), I32(m), _p(x), _p(_h(alpha)), _p(out))
    return out


def arith_element_add(x, y):
    x = _h(x); y = _h(y)
    out = np.empty_like(x)
    lib().o_arith_element_add(I64(x.size), _p(x), _p(y), _p(out))
    return out


def mask(x, mask, value):
    x = _h(x); b, n, m = x.shape
    mask = np.ascontiguousarray(mask).view(np.int8)
    assert mask.shape == (b, m)
    out = np.empty_like(x)
    lib().o_mask(I32(b), I32(n), I32(m), _p(x), _p(mask), F32(value), _p(out))
    return out


if __name__ == "__main__":
    print(build(force=True))
