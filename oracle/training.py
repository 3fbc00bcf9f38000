"""CPU oracle, second part -- TEST INFRASTRUCTURE ONLY (see oracle/__init__.py for who may import it).

numpy restatements of the reference's training-side and helper kernels.  Elementwise fp16
arithmetic is restated exactly (float64 holds every sum/product of two fp16 values exactly, so one
cast to float16 reproduces the single rounding of __hadd2/__hmul2/__hfma2); anything that sums many
terms is accumulated in float64, i.e. it is the value the reference's fp32 block reductions
approximate, and tests compare within a tolerance rather than bit for bit.

Pinned by tests/test_oracle.py against independent routes: torch.autograd gradients of the forward
formulas (gelu, softmax, both layer norms, position bias, embedding), numpy scatter-add for the two
embedding stages, and closed forms for the fp16 elementwise family.
"""
import numpy as np

f16, f32, f64 = np.float16, np.float32, np.float64


def _h(a):
    a = np.asarray(a)
    assert a.dtype == f16, a.dtype
    return a


# ---- cuda/arith.cu ---------------------------------------------------------------------------
def arith_global_scale(x, scale):
    """arith.cu:6-16: half(float(x) * scale)."""
    return (_h(x).astype(f32) * f32(scale)).astype(f16)


def arith_element_mul(x, y):
    """arith.cu:33-44: __hmul2."""
    return (_h(x).astype(f64) * _h(y).astype(f64)).astype(f16)


def arith_batch_add_forward(x, y):
    """arith.cu:47-58: x (batch, n) + y (n)."""
    return (_h(x).astype(f64) + _h(y).astype(f64)[None, :]).astype(f16)


def arith_batch_add_backward(grad_out):
    """arith.cu:61-77: column sums of (batch, n)."""
    return _h(grad_out).astype(f64).sum(0)


def arith_ln_add(x, beta):
    """arith.cu:80-94."""
    return (_h(x).astype(f64) + _h(beta).astype(f64)[None, :, None]).astype(f16)


def arith_ln_div(x, alpha):
    """arith.cu:131-143: __hmul2(x, __hdiv(1, alpha)) -- the reciprocal is rounded to fp16 first."""
    with np.errstate(divide="ignore", invalid="ignore"):
        r = (1.0 / _h(alpha).astype(f64)).astype(f16)
    return (_h(x).astype(f64) * r.astype(f64)[None, :, None]).astype(f16)


def arith_ln_sub_div(x, alpha, beta):
    """arith.cu:146-165: rev = float(1.0 / alpha) (double divide), nb = -beta * rev (fp32),
    out = __hfma2(x, half(rev), half(nb))."""
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        rev = (1.0 / _h(alpha).astype(f64)).astype(f32)
        nb = -(_h(beta).astype(f32)) * rev
        a = rev.astype(f16).astype(f64)[None, :, None]
        b = nb.astype(f16).astype(f64)[None, :, None]
        return (_h(x).astype(f64) * a + b).astype(f16)


def arith_ln_mul_backward(x, grad_out):
    """arith.cu:168-214: sum over batch and the last dim of x * grad_out."""
    return (_h(x).astype(f64) * _h(grad_out).astype(f64)).sum((0, 2))


def arith_ln_add_backward(grad_out):
    """arith.cu:217-261."""
    return _h(grad_out).astype(f64).sum((0, 2))


def arith_batch_mul_add(x, alpha, beta):
    """arith.cu:264-275: __hfma2(x, alpha[col], beta[col])."""
    return (_h(x).astype(f64) * _h(alpha).astype(f64)[None, :] + _h(beta).astype(f64)[None, :]).astype(f16)


def arith_batch_mul(x, alpha):
    """arith.cu:278-288."""
    return (_h(x).astype(f64) * _h(alpha).astype(f64)[None, :]).astype(f16)


# ---- cuda/gelu.cu:20-45 ----------------------------------------------------------------------
def gelu_backward(grad_out, x):
    """Derivative of the tanh form with the reference's literals, 0/1 outside |x| < 5 (float64)."""
    g = _h(grad_out).astype(f64)
    x = _h(x).astype(f64)
    x3 = x * x * x
    u = 0.797885 * x + 0.0356774 * x3
    d = 0.5 + (0.398942 * x + 0.0535161 * x3) / np.cosh(u) ** 2 + 0.5 * np.tanh(u)
    d = np.where((x > -5) & (x < 5), d, np.where(x < 0, 0.0, 1.0))
    return d * g


# ---- cuda/softmax.cu:86-114 ------------------------------------------------------------------
def softmax_backward(out, grad_out):
    o = _h(out).astype(f64)
    g = _h(grad_out).astype(f64)
    return o * (g - (o * g).sum(1, keepdims=True))


# ---- cuda/layernorm.cu:142-339 ---------------------------------------------------------------
def layernorm_forward_v(x, eps):
    """-> out, var where var = rsqrt(mean(x^2) + eps), shape (batch, m)."""
    x = _h(x).astype(f64)
    v = 1.0 / np.sqrt((x * x).mean(1) + eps)
    return x * v[:, None, :], v


def layernorm_forward_mv(x, eps):
    """-> out, mean, var with var = rsqrt(E[x^2] - mean^2 + eps)."""
    x = _h(x).astype(f64)
    mean = x.mean(1)
    v = 1.0 / np.sqrt((x * x).mean(1) - mean * mean + eps)
    return (x - mean[:, None, :]) * v[:, None, :], mean, v


def layernorm_backward_v(x, grad_out, var):
    """layernorm.cu:244-282 from the fp16 var the forward pass stored."""
    x = _h(x).astype(f64); g = _h(grad_out).astype(f64); v = _h(var).astype(f64)[:, None, :]
    n = x.shape[1]
    gv = (g * (-0.5 * v ** 3) * x).sum(1, keepdims=True)
    return g * v + gv * x * 2.0 / n


def layernorm_backward_mv(x, grad_out, mean, var):
    """layernorm.cu:285-339 (terms exactly as the kernel forms them)."""
    x = _h(x).astype(f64); g = _h(grad_out).astype(f64)
    mu = _h(mean).astype(f64)[:, None, :]; v = _h(var).astype(f64)[:, None, :]
    n = x.shape[1]
    gv = (g * (-0.5 * v ** 3) * (x - mu)).sum(1, keepdims=True)
    gm = (-g * v).sum(1, keepdims=True) - 2.0 * gv * mu
    return g * v + (gm + gv * x * 2.0) / n


# ---- cuda/gemm.cu:102-172 --------------------------------------------------------------------
def _round_i8(q):
    q = np.rint(q)
    q = np.where(np.isnan(q), 0.0, q)
    return np.clip(q, -128, 127).astype(np.int8)


def gemm_backward_round_scale(mat, scale_y, broad_cast_y):
    """-> int8 (batch, n, m), scale_x fp16 (batch, n).  The row maximum of |mat * scale_y| (fp32
    product) divided by the double 127.0 and stored as float is the divisor of the rounding; its
    fp16 rounding is what scale_x receives."""
    p = _h(mat).astype(f32) * (_h(scale_y).astype(f32)[None, None, :] if broad_cast_y else _h(scale_y).astype(f32)[:, None, :])
    s = (np.abs(p).max(2).astype(f64) / 127.0).astype(f32)
    with np.errstate(divide="ignore", invalid="ignore"):
        q = _round_i8(p / s[:, :, None])
    return q, s.astype(f16)


def gemm_backward_scale_round(mat, scale_x, broad_cast_x):
    """The same along dim 1 -> int8, scale_y fp16 (batch, m)."""
    p = _h(mat).astype(f32) * (_h(scale_x).astype(f32)[None, :, None] if broad_cast_x else _h(scale_x).astype(f32)[:, :, None])
    s = (np.abs(p).max(1).astype(f64) / 127.0).astype(f32)
    with np.errstate(divide="ignore", invalid="ignore"):
        q = _round_i8(p / s[:, None, :])
    return q, s.astype(f16)


# ---- cuda/position_bucket.cu:57-103 ----------------------------------------------------------
def position_embedding_backward(query_len, key_len, num_buckets, max_distance, mapping, grad_out, bidirectional):
    g = _h(grad_out).astype(f64)
    heads = g.shape[0]
    q = np.arange(query_len)[None, :]; k = np.arange(key_len)[:, None]
    rel = q - k
    off = np.zeros_like(rel)
    if bidirectional:
        off = np.where(rel < 0, num_buckets // 2, 0)
        rel = np.abs(rel)
    else:
        rel = np.maximum(rel, 0)
    rel = np.minimum(rel, max_distance - 1)
    bucket = np.asarray(mapping)[rel] + off
    out = np.zeros((heads, num_buckets), f64)
    for h in range(heads):
        out[h] = np.bincount(bucket.ravel(), weights=g[h].ravel(), minlength=num_buckets)
    return out


# ---- cuda/embedding.cu:36-88 -----------------------------------------------------------------
def embedding_backward_stage1(grad_out, argsort_ids, sorted_ids, grad):
    """Sequential restatement (fp32 running sums in id order, like the kernel's per-column loop).
    grad is updated in place for complete runs; returns aux_grad (batch, m) fp16 and aux_idx."""
    go = _h(grad_out).astype(f32)
    batch, n = sorted_ids.shape
    m = go.shape[1]
    aux = np.zeros((batch, m), f16)
    aux_idx = np.zeros((batch,), np.int32)
    for b in range(batch):
        s = np.zeros((m,), f32)
        for i in range(n):
            s = s + go[argsort_ids[b, i]]
            if i + 1 == n:
                aux[b] = s.astype(f16)
                aux_idx[b] = sorted_ids[b, i]
            elif sorted_ids[b, i] != sorted_ids[b, i + 1]:
                grad[sorted_ids[b, i]] = s.astype(f16)
                s = np.zeros((m,), f32)
    return aux, aux_idx


def embedding_backward_stage2(aux_grad, aux_idx, grad):
    aux = _h(aux_grad).astype(f32)
    batch = aux.shape[0]
    s = np.zeros((aux.shape[1],), f32)
    for i in range(batch):
        s = s + aux[i]
        if i + 1 == batch or aux_idx[i] != aux_idx[i + 1]:
            grad[aux_idx[i]] = (grad[aux_idx[i]].astype(f32) + s).astype(f16)
            s = np.zeros_like(s)
    return grad


# ---- cuda/utils.cu:38-54 ---------------------------------------------------------------------
def adjustify_logits(logits, temperature, frequency_penalty, presence_penalty, frequency):
    v = _h(logits).astype(f32) / f32(temperature)
    freq = np.asarray(frequency)
    v = v - f32(frequency_penalty) * freq.astype(f32)
    v = v - f32(presence_penalty) * (freq > 0).astype(f32)
    return v.astype(f16)
