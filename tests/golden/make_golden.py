"""Writes tests/golden/path_vectors.npz: small input/output vectors for every kernel family on the path.

Inputs are the closed-form generators the reference's own tests use, so they need no random-number
generator: 0.4*sin / 0.4*cos / 0.4*sin over ranges 9, 7, 5 for attention (test_coopmat_attention.jl:54-55),
0.4*sin over 9 and 0.3*cos over 7 for convolution and GEMM operands (test_convtranspose_gemm.jl:170-173).
Each case stores the fp16 inputs, the oracle's output (``*_oracle``: what the CPU restatement of the
reference's algorithm returns, frozen here so that a later change to the oracle shows up as a diff) and an
independent float64 closed form computed below with numpy alone (``*_f64``, stored as float32).

Run from the repo root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "path_vectors.npz")


def wave(fn, amp, span, shape):
    n = int(np.prod(shape))
    return (amp * fn(np.linspace(0.0, span, n))).astype(np.float16).reshape(shape)


def gelu_erf64(x):
    from math import erf
    return 0.5 * x * (1.0 + np.vectorize(erf)(x / np.sqrt(2.0)))


def softmax_attention64(q, k, v, scale, kv_len=None):
    q, k, v = (a.astype(np.float64) for a in (q, k, v))
    s = np.einsum("bhqe,bhke->bhqk", q, k) * scale
    if kv_len is not None:
        for b, n in enumerate(kv_len):
            s[b, :, :, n:] = -np.inf
    s -= s.max(axis=-1, keepdims=True)
    p = np.exp(s)
    p /= p.sum(axis=-1, keepdims=True)
    return np.einsum("bhqk,bhke->bhqe", p, v)


def conv64(x, w, b, stride, padding, dilation):
    """Direct convolution, (y, x) pairs, groups = 1."""
    x, w = x.astype(np.float64), w.astype(np.float64)
    N, C, H, W = x.shape
    Co, _, KH, KW = w.shape
    OH = (H + 2 * padding[0] - dilation[0] * (KH - 1) - 1) // stride[0] + 1
    OW = (W + 2 * padding[1] - dilation[1] * (KW - 1) - 1) // stride[1] + 1
    xp = np.zeros((N, C, H + 2 * padding[0], W + 2 * padding[1]))
    xp[:, :, padding[0]:padding[0] + H, padding[1]:padding[1] + W] = x
    out = np.zeros((N, Co, OH, OW))
    for kh in range(KH):
        for kw in range(KW):
            patch = xp[:, :, kh * dilation[0]:kh * dilation[0] + stride[0] * (OH - 1) + 1:stride[0],
                       kw * dilation[1]:kw * dilation[1] + stride[1] * (OW - 1) + 1:stride[1]]
            out += np.einsum("nchw,oc->nohw", patch, w[:, :, kh, kw])
    return out + (0.0 if b is None else b.astype(np.float64)[None, :, None, None])


def convtranspose64(x, w, b, stride):
    """Transposed convolution with no padding or dilation, groups = 1; w is (Cin, Cout, KH, KW)."""
    x, w = x.astype(np.float64), w.astype(np.float64)
    N, C, H, W = x.shape
    _, Co, KH, KW = w.shape
    out = np.zeros((N, Co, (H - 1) * stride[0] + KH, (W - 1) * stride[1] + KW))
    for kh in range(KH):
        for kw in range(KW):
            out[:, :, kh:kh + stride[0] * (H - 1) + 1:stride[0], kw:kw + stride[1] * (W - 1) + 1:stride[1]] += \
                np.einsum("nchw,co->nohw", x, w[:, :, kh, kw])
    return out + b.astype(np.float64)[None, :, None, None]


def main():
    z = {}
    # ---- linear: bias seeds the accumulator, GELU(erf) on the rounded sum (matmul.jl:17-27, 210-214)
    X, Wt, bias = wave(np.sin, 0.4, 9, (70, 96)), wave(np.cos, 0.3, 7, (96, 136)), wave(np.sin, 0.4, 5, (136,))
    z["gemm_x"], z["gemm_w"], z["gemm_bias"] = X, Wt, bias
    z["gemm_oracle"] = oracle.gemm_f16(X, Wt, bias)
    z["gemm_f64"] = (X.astype(np.float64) @ Wt.astype(np.float64) + bias.astype(np.float64)).astype(np.float32)
    z["gemm_gelu_oracle"] = oracle.gemm_f16(X, Wt, bias, epi="gelu")
    z["gemm_gelu_f64"] = gelu_erf64(z["gemm_oracle"].astype(np.float64)).astype(np.float32)      # on the ROUNDED sum
    # ---- attention, the reference's (E,L,H,B) = (64,256,2,1) at L = 128, and a ragged head-72 case with masked keys
    for tag, (B, H, Lq, Lk, E), kv_len in (("attn", (1, 2, 128, 128, 64), None), ("attn72", (2, 2, 70, 77, 72), [77, 31])):
        q, k, v = wave(np.sin, 0.4, 9, (B, H, Lq, E)), wave(np.cos, 0.4, 7, (B, H, Lk, E)), wave(np.sin, 0.4, 5, (B, H, Lk, E))
        z[tag + "_q"], z[tag + "_k"], z[tag + "_v"] = q, k, v
        kl = None if kv_len is None else np.asarray(kv_len, dtype=np.int32)
        if kl is not None:
            z[tag + "_kv_len"] = kl
        z[tag + "_oracle"] = oracle.sdpa_threepass_f16(q, k, v, kv_len=kl)
        z[tag + "_f64"] = softmax_attention64(q, k, v, 1.0 / np.sqrt(E), kv_len).astype(np.float32)
    # ---- convolution: 3x3 stride 1 pad 1 and 5x5 stride 2 pad 2 (the shapes of test_convtranspose_gemm.jl:188-191, scaled)
    for tag, (N, C, H, W, Co, K, s, p) in (("conv3", (1, 16, 24, 24, 24, 3, 1, 1)), ("conv5", (2, 7, 20, 20, 12, 5, 2, 2))):
        x, w, b = wave(np.sin, 0.4, 9, (N, C, H, W)), wave(np.cos, 0.3, 7, (Co, C, K, K)), wave(np.sin, 0.4, 5, (Co,))
        z[tag + "_x"], z[tag + "_w"], z[tag + "_bias"] = x, w, b
        z[tag + "_geom"] = np.asarray([s, p], dtype=np.int64)
        z[tag + "_oracle"] = oracle.conv2d_f16(x, w, b, (s, s), (p, p))
        z[tag + "_f64"] = conv64(x, w, b, (s, s), (p, p), (1, 1)).astype(np.float32)
    # ---- transposed convolution, kernel = stride = 2 (SAM 2's upsampler shape, test_convtranspose_gemm.jl:36, scaled)
    x, w, b = wave(np.sin, 0.4, 9, (1, 16, 8, 8)), wave(np.cos, 0.3, 7, (16, 8, 2, 2)), wave(np.sin, 0.4, 5, (8,))
    z["convt_x"], z["convt_w"], z["convt_bias"] = x, w, b
    z["convt_oracle"] = oracle.convtranspose2d_f16(x, w, b, (2, 2))
    z["convt_f64"] = convtranspose64(x, w, b, (2, 2)).astype(np.float32)
    # ---- layer norm over the last axis, eps 1e-6, affine (layernorm.jl:53-113)
    a, g, bt = wave(np.sin, 2.0, 9, (5, 384)), wave(np.cos, 1.0, 7, (384,)), wave(np.sin, 0.4, 5, (384,))
    z["ln_a"], z["ln_gamma"], z["ln_beta"] = a, g, bt
    out, mean, rstd = oracle.layernorm_f16(a, g, bt, eps=1e-6)
    z["ln_oracle"], z["ln_mean_oracle"], z["ln_rstd_oracle"] = out, mean, rstd
    a64 = a.astype(np.float64)
    mu, var = a64.mean(axis=1, keepdims=True), a64.var(axis=1, keepdims=True)
    z["ln_f64"] = ((a64 - mu) / np.sqrt(var + 1e-6) * g.astype(np.float64) + bt.astype(np.float64)).astype(np.float32)
    np.savez_compressed(OUT, **z)
    print(f"wrote {OUT}: {len(z)} arrays, {os.path.getsize(OUT)} bytes")


if __name__ == "__main__":
    main()
