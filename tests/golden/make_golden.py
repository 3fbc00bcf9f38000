"""Writes tests/golden/path_small.npz: seeded inputs and expected outputs of the int8 path for
a small case, computed with numpy closed forms and Python integers only (no oracle code, no
product code, no reference code).  The reference ships no golden vectors for this path (its
tests draw unseeded random inputs and compare on the GPU), so the fixtures restate the closed
forms of its kernels:
  scale  = fp16( fp32(max|x|) / 127 )                       cuda/gemm.cu:60-98
  q      = int8( rint( fp32(x) / fp32(scale) ) )            cuda/gemm.cu:6-33
  acc    = integer matrix product                           kernels/gemm.py:127-186
  out    = fp16( (fp32(acc) * sx) * sy )                    cuda/gemm.cu:37-57
  bucket = T5 relative position bucket, exact integer form  cuda/position_bucket.cu:6-21
  ln / softmax / gelu = float64 textbook forms rounded to fp16 (tolerance fixtures)

    python tests/golden/make_golden.py
"""
import os

import numpy as np

f16, f32, f64 = np.float16, np.float32, np.float64


def scale(absmax):
    return (absmax.astype(f32) / f32(127)).astype(f16)


def rnd(x, s):
    d = x.astype(f32) / s.astype(f32)
    return np.clip(np.rint(d), -128, 127).astype(np.int8)


def bucket_table(num_buckets, max_distance, bidirectional):
    part = num_buckets // (2 if bidirectional else 1)
    E = part // 2; L = part - E; R = max_distance // E
    out = []
    for i in range(max_distance):
        if i < E:
            out.append(i)
        else:
            j = 0
            while (R ** (j + 1)) * (E ** L) <= i ** L:
                j += 1
            out.append(j + E)
    return np.array(out, np.int32)


def main():
    rng = np.random.default_rng(20240521)
    M, K, N = 24, 64, 40
    a = rng.standard_normal((1, M, K)).astype(f16)
    w = (rng.standard_normal((1, N, K)) * 0.02).astype(f16)
    a_scale = scale(np.abs(a).max(-1)); w_scale = scale(np.abs(w).max(-1))
    a_q = rnd(a, a_scale[..., None]); w_q = rnd(w, w_scale[..., None])
    acc = np.zeros((1, M, N), np.int64)
    for i in range(M):
        for j in range(N):
            acc[0, i, j] = sum(int(x) * int(y) for x, y in zip(a_q[0, i], w_q[0, j]))
    acc = acc.astype(np.int32)
    out = ((acc.astype(f32) * a_scale.astype(f32)[0][None, :, None]) * w_scale.astype(f32)[0][None, None, :]).astype(f16)
    a_scale_t = scale(np.abs(a).max(1)); a_q_t = rnd(a, a_scale_t[:, None, :])
    x = (rng.standard_normal((2, 48, 16)) * 2).astype(f16)
    xf = x.astype(f64)
    mean = xf.mean(1, keepdims=True); var = (xf ** 2).mean(1, keepdims=True) - mean ** 2
    ln = ((xf - mean) / np.sqrt(var + 1e-5)).astype(f16)
    e = np.exp(xf - xf.max(1, keepdims=True)); sm = (e / e.sum(1, keepdims=True)).astype(f16)
    gelu = (0.5 * xf * (1.0 + np.tanh(0.7978845608028654 * xf * (1.0 + 0.044715 * xf * xf)))).astype(f16)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "path_small.npz")
    np.savez_compressed(path, a=a, w=w, a_scale=a_scale, w_scale=w_scale, a_q=a_q, w_q=w_q, acc=acc, out=out,
                        a_scale_t=a_scale_t, a_q_t=a_q_t, x=x, ln=ln, softmax=sm, gelu=gelu,
                        pos_table_32_128_bidi=bucket_table(32, 128, True),
                        pos_table_32_128_uni=bucket_table(32, 128, False))
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
