"""ctypes front end of the CPU oracle (``oracle.c``).  TEST INFRASTRUCTURE ONLY.

Only tests, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg may
import this package; the product package ``juliavision_amd`` never does.

Arrays follow the reference's reversed-layout rule (DNNKernels/src/safetensors.jl:7-12):
a Julia ``(E, L, H, B)`` array is the C-contiguous numpy array of shape ``(B, H, L, E)``.
fp16 data is ``numpy.float16``.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

EPI = {"none": 0, "gelu": 1, "gelu_erf": 1, "gelu_tanh": 2, "relu": 3}


def build(force: bool = False) -> str:
    """Compile ``oracle.c`` with gcc (``make -C oracle``)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)
    return _LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.orc_erf.restype = C.c_float
        _lib.orc_erf.argtypes = [C.c_float]
        _lib.orc_convsize.restype = C.c_int64
        _lib.orc_convsize.argtypes = [C.c_int64] * 5
        _lib.orc_threads.restype = C.c_int
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _i64(x):
    return C.c_int64(int(x))


def _strides(a: np.ndarray):
    """Element strides of a (B,H,L,E)-shaped numpy view in (E,L,H,B) order."""
    it = a.itemsize
    s = [a.strides[3] // it, a.strides[2] // it, a.strides[1] // it, a.strides[0] // it]
    return (C.c_int64 * 4)(*s)


def threads() -> int:
    return int(lib().orc_threads())


# ----------------------------------------------------------------------------- seeded inputs

def randn_f16(shape, seed: int, mean: float = 0.0, std: float = 1.0) -> np.ndarray:
    out = np.empty(shape, dtype=np.float16)
    lib().orc_randn_f16(_p(out), _i64(out.size), C.c_uint64(seed), C.c_double(mean), C.c_double(std))
    return out


def randn_f32(shape, seed: int, mean: float = 0.0, std: float = 1.0) -> np.ndarray:
    out = np.empty(shape, dtype=np.float32)
    lib().orc_randn_f32(_p(out), _i64(out.size), C.c_uint64(seed), C.c_double(mean), C.c_double(std))
    return out


def uniform_f16(shape, seed: int, lo: float = 0.0, hi: float = 1.0) -> np.ndarray:
    out = np.empty(shape, dtype=np.float16)
    lib().orc_uniform_f16(_p(out), _i64(out.size), C.c_uint64(seed), C.c_double(lo), C.c_double(hi))
    return out


# ----------------------------------------------------------------------------- activations

def erf_scalar(x: float) -> float:
    return float(lib().orc_erf(C.c_float(x)))


def act_f16(a: np.ndarray, kind: str) -> np.ndarray:
    """kind in {'erf','gelu','gelu_tanh','relu'}; evaluated in fp32, rounded once."""
    code = {"erf": 0, "gelu": 1, "gelu_tanh": 2, "relu": 3}[kind]
    a = np.ascontiguousarray(a, dtype=np.float16)
    out = np.empty_like(a)
    lib().orc_act_f16(_p(out), _p(a), _i64(a.size), C.c_int(code))
    return out


# ----------------------------------------------------------------------------- GEMM

def gemm_f16(X, W, bias=None, *, w_layout="kf", bias_mode=None, epi="none", out_f32=False, residual=None):
    """Y[T,F] = X[T,K] . W (+bias) in the mm2 form.  X, W may be 2-D or 3-D (batched)."""
    X = np.ascontiguousarray(X, dtype=np.float16)
    W = np.ascontiguousarray(W, dtype=np.float16)
    batched = X.ndim == 3 or W.ndim == 3
    nb = max(X.shape[0] if X.ndim == 3 else 1, W.shape[0] if W.ndim == 3 else 1)
    T, K = X.shape[-2:]
    if w_layout == "kf":
        assert W.shape[-2] == K
        F = W.shape[-1]
    else:
        assert W.shape[-1] == K
        F = W.shape[-2]
    Y = np.empty((nb, T, F) if batched else (T, F), dtype=np.float32 if out_f32 else np.float16)
    if bias is not None:
        bias = np.ascontiguousarray(bias, dtype=np.float16)
        if bias_mode is None:
            bias_mode = "col"
    bm = {None: 0, "none": 0, "col": 1, "row": 2}[bias_mode]
    if residual is not None:
        residual = np.ascontiguousarray(residual, dtype=np.float16)
        assert residual.shape == Y.shape
    lib().orc_gemm_f16(_p(Y), _p(X), _p(W), _p(bias), _p(residual),
                       _i64(T), _i64(K), _i64(F), _i64(F), _i64(K), _i64(W.shape[-1]),
                       C.c_int(0 if w_layout == "kf" else 1), C.c_int(bm), C.c_int(EPI[epi]),
                       C.c_int(1 if out_f32 else 0), _i64(nb), _i64(T * F),
                       _i64(T * K if X.ndim == 3 else 0), _i64(W.shape[-2] * W.shape[-1] if W.ndim == 3 else 0))
    return Y


# ----------------------------------------------------------------------------- attention

def _bias_args(bias, Lk, Lq, H, B):
    if bias is None:
        return None, 0, (C.c_int64 * 4)(0, 0, 0, 0), None
    assert bias.ndim == 4, "bias is (B|1, H|1, Lq|1, Lk|1) in numpy order"
    keep = bias
    bias = np.ascontiguousarray(bias)
    it = bias.itemsize
    full = (B, H, Lq, Lk)
    st = []
    for ax in (3, 2, 1, 0):  # (Lk, Lq, H, B) order
        assert bias.shape[ax] in (1, full[ax])
        st.append(0 if bias.shape[ax] == 1 else bias.strides[ax] // it)
    return bias, (1 if bias.dtype == np.float32 else 0), (C.c_int64 * 4)(*st), keep


def _sdpa_common(fn, out, q, k, v, bias, kv_len, scale, extra_first=()):
    B, H, Lq, E = q.shape
    Lk = k.shape[2]
    scale = (1.0 / np.sqrt(E)) if scale is None else scale
    b_arr, b_f32, b_st, _ = _bias_args(bias, Lk, Lq, H, B)
    kl = None if kv_len is None else np.ascontiguousarray(kv_len, dtype=np.int32)
    fn(*extra_first, _p(q), _strides(q), _p(k), _strides(k), _p(v), _strides(v),
       _p(b_arr), C.c_int(b_f32), b_st, _p(kl),
       _i64(E), _i64(Lq), _i64(Lk), _i64(H), _i64(B), C.c_float(scale))
    return out


def sdpa_threepass_f16(q, k, v, bias=None, scale=None, *, kv_len=None, out_f32=False):
    """q,k,v: float16 numpy views of shape (B,H,L,E) (any strides). Returns (B,H,Lq,E)."""
    assert q.dtype == k.dtype == v.dtype == np.float16
    B, H, Lq, E = q.shape
    out = np.empty((B, H, Lq, E), dtype=np.float32 if out_f32 else np.float16)
    return _sdpa_common(lib().orc_sdpa_threepass_f16, out, q, k, v, bias, kv_len, scale,
                        extra_first=(_p(out), C.c_int(1 if out_f32 else 0)))


def sdpa_ref_f32(q, k, v, bias=None, scale=None, *, kv_len=None):
    assert q.dtype == k.dtype == v.dtype == np.float16
    B, H, Lq, E = q.shape
    out = np.empty((B, H, Lq, E), dtype=np.float32)
    return _sdpa_common(lib().orc_sdpa_ref_f32, out, q, k, v, bias, kv_len, scale, extra_first=(_p(out),))


def sdpa_flash_f32(q, k, v, scale=None, *, bk=32, nsplit=1):
    q, k, v = (np.ascontiguousarray(a, dtype=np.float16) for a in (q, k, v))
    B, H, Lq, E = q.shape
    Lk = k.shape[2]
    scale = (1.0 / np.sqrt(E)) if scale is None else scale
    out = np.empty((B, H, Lq, E), dtype=np.float32)
    lib().orc_sdpa_flash_f32(_p(out), _p(q), _p(k), _p(v), _i64(E), _i64(Lq), _i64(Lk), _i64(H), _i64(B),
                             C.c_float(scale), _i64(bk), _i64(nsplit))
    return out


# ----------------------------------------------------------------------------- convolution

def convsize(n, k, s, p, d):
    return int(lib().orc_convsize(_i64(n), _i64(k), _i64(s), _i64(p), _i64(d)))


def conv2d_f16(x, w, bias=None, stride=(1, 1), padding=(0, 0), dilation=(1, 1), groups=1, relu=False, out_f32=False):
    """x: (N,Cin,H,W) fp16; w: (Cout,Cin/g,KH,KW); stride/padding/dilation are (y, x) pairs as in torch."""
    x = np.ascontiguousarray(x, dtype=np.float16)
    w = np.ascontiguousarray(w, dtype=np.float16)
    N, Cin, Hi, Wi = x.shape
    Cout, _, KH, KW = w.shape
    OH = convsize(Hi, KH, stride[0], padding[0], dilation[0])
    OW = convsize(Wi, KW, stride[1], padding[1], dilation[1])
    out = np.empty((N, Cout, OH, OW), dtype=np.float32 if out_f32 else np.float16)
    if bias is not None:
        bias = np.ascontiguousarray(bias, dtype=np.float16)
    lib().orc_conv2d_f16(_p(out), C.c_int(1 if out_f32 else 0), _p(x), _p(w), _p(bias),
                         _i64(Wi), _i64(Hi), _i64(Cin), _i64(N), _i64(KW), _i64(KH), _i64(Cout),
                         _i64(stride[1]), _i64(stride[0]), _i64(padding[1]), _i64(padding[0]),
                         _i64(dilation[1]), _i64(dilation[0]), _i64(groups), C.c_int(1 if relu else 0))
    return out


def convtransposesize(n, k, s, p, d, op):
    return int(lib().orc_convtransposesize(_i64(n), _i64(k), _i64(s), _i64(p), _i64(d), _i64(op)))


def convtranspose2d_f16(x, w, bias=None, stride=(1, 1), padding=(0, 0), dilation=(1, 1), output_padding=(0, 0), groups=1, out_f32=False):
    """x: (N,Cin,H,W) fp16; w: (Cin,Cout/g,KH,KW) (torch's transposed-convolution weight); pairs are (y, x) as in torch."""
    x = np.ascontiguousarray(x, dtype=np.float16)
    w = np.ascontiguousarray(w, dtype=np.float16)
    N, Cin, Hi, Wi = x.shape
    _, coutg, KH, KW = w.shape
    Cout = coutg * groups
    OH = convtransposesize(Hi, KH, stride[0], padding[0], dilation[0], output_padding[0])
    OW = convtransposesize(Wi, KW, stride[1], padding[1], dilation[1], output_padding[1])
    out = np.empty((N, Cout, OH, OW), dtype=np.float32 if out_f32 else np.float16)
    if bias is not None:
        bias = np.ascontiguousarray(bias, dtype=np.float16)
    lib().orc_convtranspose2d_f16(_p(out), C.c_int(1 if out_f32 else 0), _p(x), _p(w), _p(bias),
                                  _i64(Wi), _i64(Hi), _i64(Cin), _i64(N), _i64(KW), _i64(KH), _i64(Cout),
                                  _i64(stride[1]), _i64(stride[0]), _i64(padding[1]), _i64(padding[0]),
                                  _i64(dilation[1]), _i64(dilation[0]), _i64(output_padding[1]), _i64(output_padding[0]), _i64(groups))
    return out


def im2col_f16(x, KH, KW, stride=(1, 1), padding=(0, 0), dilation=(1, 1), MP=None, CRSP=None):
    """Returns col as row-major [CRSP][MP] (= the reference's column-major MP x CRSP)."""
    x = np.ascontiguousarray(x, dtype=np.float16)
    N, Cin, Hi, Wi = x.shape
    OH = convsize(Hi, KH, stride[0], padding[0], dilation[0])
    OW = convsize(Wi, KW, stride[1], padding[1], dilation[1])
    MP = N * OH * OW if MP is None else MP
    CRSP = Cin * KH * KW if CRSP is None else CRSP
    col = np.empty((CRSP, MP), dtype=np.float16)
    lib().orc_im2col_f16(_p(col), _p(x), _i64(Wi), _i64(Hi), _i64(Cin), _i64(N), _i64(KW), _i64(KH),
                         _i64(stride[1]), _i64(stride[0]), _i64(padding[1]), _i64(padding[0]),
                         _i64(dilation[1]), _i64(dilation[0]), _i64(MP), _i64(CRSP))
    return col


# ----------------------------------------------------------------------------- layer norm, add

def layernorm_f16(a, gamma=None, beta=None, eps=1e-5):
    a = np.ascontiguousarray(a, dtype=np.float16)
    Cn = a.shape[-1]
    groups = a.size // Cn
    out = np.empty_like(a)
    mean = np.empty(groups, dtype=np.float32)
    rstd = np.empty(groups, dtype=np.float32)
    g = None if gamma is None else np.ascontiguousarray(gamma, dtype=np.float16)
    b = None if beta is None else np.ascontiguousarray(beta, dtype=np.float16)
    lib().orc_layernorm_f16(_p(out), _p(mean), _p(rstd), _p(a), _p(g), _p(b), _i64(Cn), _i64(groups), C.c_float(eps))
    return out, mean, rstd


def softmax_f16(a, scale: float = 1.0):
    """Softmax over the last axis, fp16 in and out (softmax_kernel!, ops.jl:474-555)."""
    a = np.ascontiguousarray(a, dtype=np.float16)
    out = np.empty_like(a)
    n = a.shape[-1]
    lib().orc_softmax_f16(_p(out), _p(a), _i64(n), _i64(a.size // max(n, 1)), C.c_float(scale))
    return out


def scale_f16(a, c: float):
    a = np.ascontiguousarray(a, dtype=np.float16)
    out = np.empty_like(a)
    lib().orc_scale_f16(_p(out), _p(a), C.c_float(c), _i64(a.size))
    return out


def add_f16(a, b):
    a = np.ascontiguousarray(a, dtype=np.float16)
    b = np.ascontiguousarray(b, dtype=np.float16)
    out = np.empty_like(a)
    lib().orc_add_f16(_p(out), _p(a), _p(b), _i64(a.size))
    return out


# ----------------------------------------------------------------------------- the parity metrics

def max_rel(got, want) -> float:
    """max|a-b| / max|b|  (the gate BASELINE names: <= 1e-2)."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    d = float(np.max(np.abs(got - want))) if got.size else 0.0
    m = float(np.max(np.abs(want))) if want.size else 0.0
    return d / m if m > 0 else d


def cosine(got, want) -> float:
    a = np.asarray(got, dtype=np.float64).ravel()
    b = np.asarray(want, dtype=np.float64).ravel()
    na, nb = np.linalg.norm(a), np.linalg.norm(b)
    if na == 0 and nb == 0:
        return 1.0
    return float(a @ b / (na * nb))
