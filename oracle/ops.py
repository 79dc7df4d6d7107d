"""TEST INFRASTRUCTURE ONLY: numpy-facing loader of the C oracle (oracle/ops_ref.c)."""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libops_ref.so")
_lib = None
_F = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
_I = np.ctypeslib.ndpointer(dtype=np.int64, flags="C_CONTIGUOUS")


def build():
    subprocess.check_call(["make", "-C", _HERE, "-s"])


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = C.CDLL(_SO)
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def gemm(X, Y, M, N, K, xs_r, xs_k, ys_c, ys_k, ldc, alpha=1.0, beta=0.0, C_in=None):
    """X, Y flat float32 buffers; returns flat C of size (M-1)*ldc + N."""
    X, Y = _f32(X).ravel(), _f32(Y).ravel()
    out = np.zeros((M - 1) * ldc + N, np.float32) if C_in is None else _f32(C_in).ravel().copy()
    lib().ref_gemm(_p(X), _p(Y), _p(out), C.c_long(M), C.c_long(N), C.c_long(K), C.c_long(xs_r), C.c_long(xs_k),
                   C.c_long(ys_c), C.c_long(ys_k), C.c_long(ldc), C.c_float(alpha), C.c_float(beta))
    return out


def sgemm_colmajor(transa, transb, m, n, k, alpha, A, lda, B, ldb, beta, Cm, ldc):
    A, B = _f32(A).ravel(), _f32(B).ravel()
    out = _f32(Cm).ravel().copy()
    lib().ref_sgemm_colmajor(transa, transb, m, n, k, C.c_float(alpha), _p(A), lda, _p(B), ldb, C.c_float(beta),
                             _p(out), ldc)
    return out


def conv2d(x, w, stride=(1, 1), pad=(0, 0), x_nhwc=False, y_nhwc=False):
    """x: [N,C,H,W] (or [N,H,W,C] if x_nhwc); w: [K,C,R,S]."""
    x, w = _f32(x), _f32(w)
    if x_nhwc:
        N, H, W, Ci = x.shape
    else:
        N, Ci, H, W = x.shape
    Co, _, KH, KW = w.shape
    Ho = (H + 2 * pad[0] - KH) // stride[0] + 1
    Wo = (W + 2 * pad[1] - KW) // stride[1] + 1
    y = np.empty((N, Ho, Wo, Co) if y_nhwc else (N, Co, Ho, Wo), np.float32)
    lib().ref_conv2d(_p(x), _p(w), _p(y), N, H, W, Ci, Co, KH, KW, stride[0], stride[1], pad[0], pad[1],
                     int(x_nhwc), int(y_nhwc))
    return y


def bn(x, gamma, beta, mean, var, eps, C_, hw=1, nhwc=True, relu=False):
    x = _f32(x)
    y = np.empty_like(x)
    rows = x.size // C_
    lib().ref_bn(_p(x), _p(y), _p(_f32(gamma)), _p(_f32(beta)), _p(_f32(mean)), _p(_f32(var)), C.c_double(eps),
                 C.c_long(rows), C_, C.c_long(hw), int(nhwc), int(relu))
    return y


def layernorm(x, res, gamma, beta, eps):
    x = _f32(x)
    res = _f32(res)
    y = np.empty_like(x)
    width = x.shape[-1]
    lib().ref_layernorm(_p(x), _p(res), _p(_f32(gamma)), _p(_f32(beta)), _p(y), C.c_long(x.size // width), width,
                        C.c_double(eps))
    return y


def softmax(x, mask=None, scale=1.0, rows_per_mask=1):
    x = _f32(x)
    mask = _f32(mask)
    y = np.empty_like(x)
    width = x.shape[-1]
    lib().ref_softmax(_p(x), _p(mask), _p(y), C.c_long(x.size // width), width, C.c_double(scale),
                      C.c_long(rows_per_mask))
    return y


def attention(q, k, v, mask=None, scale=1.0):
    """q, k, v: [B, S, A, dh]; mask: [B, S] additive or None.  Returns [B, S, A, dh] float32:
    softmax over keys of scale * q.k + mask, times v, all in float64 (the sequence the reference
    forwards as cublasSgemmStridedBatched, softmax, cublasSgemmStridedBatched,
    include/server/cuda_server.hpp:524-550)."""
    q, k, v = (np.asarray(t, dtype=np.float64) for t in (q, k, v))
    s = np.einsum("bqad,bkad->baqk", q, k) * scale
    if mask is not None:
        s = s + np.asarray(mask, dtype=np.float64)[:, None, None, :]
    s = s - s.max(-1, keepdims=True)
    e = np.exp(s)
    pr = e / e.sum(-1, keepdims=True)
    return np.einsum("baqk,bkad->bqad", pr, v).astype(np.float32)


def depthwise_conv2d(x, w, stride=(1, 1), pad=(0, 0)):
    """x: [N,H,W,C] (NHWC), w: [C,1,KH,KW]; groups == C.  float64 accumulation, float32 result
    (cudnnConvolutionForward with a group count equal to the channel count)."""
    x = np.asarray(x, dtype=np.float64)
    w = np.asarray(w, dtype=np.float64)
    N, H, W, Cc = x.shape
    KH, KW = w.shape[2], w.shape[3]
    Ho, Wo = (H + 2 * pad[0] - KH) // stride[0] + 1, (W + 2 * pad[1] - KW) // stride[1] + 1
    xp = np.zeros((N, H + 2 * pad[0], W + 2 * pad[1], Cc))
    xp[:, pad[0]:pad[0] + H, pad[1]:pad[1] + W] = x
    y = np.zeros((N, Ho, Wo, Cc))
    for kh in range(KH):
        for kw in range(KW):
            y += xp[:, kh:kh + (Ho - 1) * stride[0] + 1:stride[0], kw:kw + (Wo - 1) * stride[1] + 1:stride[1]] * w[:, 0, kh, kw]
    return y.astype(np.float32)


def avgpool2d(x, k, stride, pad=0):
    """x: [N,H,W,C]; k x k window average with the zero padding counted in the divisor."""
    x = np.asarray(x, dtype=np.float64)
    N, H, W, Cc = x.shape
    Ho, Wo = (H + 2 * pad - k) // stride + 1, (W + 2 * pad - k) // stride + 1
    xp = np.zeros((N, H + 2 * pad, W + 2 * pad, Cc))
    xp[:, pad:pad + H, pad:pad + W] = x
    y = np.zeros((N, Ho, Wo, Cc))
    for kh in range(k):
        for kw in range(k):
            y += xp[:, kh:kh + (Ho - 1) * stride + 1:stride, kw:kw + (Wo - 1) * stride + 1:stride]
    return (y / (k * k)).astype(np.float32)


def activation(x, name):
    """relu6 / silu / sigmoid in float64 (the activations of the MobileNet / EfficientNet families)."""
    x = np.asarray(x, dtype=np.float64)
    if name == "relu6":
        return np.clip(x, 0.0, 6.0).astype(np.float32)
    if name == "silu":
        return (x / (1.0 + np.exp(-x))).astype(np.float32)
    if name == "sigmoid":
        return (1.0 / (1.0 + np.exp(-x))).astype(np.float32)
    raise ValueError(name)


def gelu(x):
    x = _f32(x)
    y = np.empty_like(x)
    lib().ref_gelu(_p(x), _p(y), C.c_long(x.size))
    return y


def maxpool(x, k, stride, pad, nhwc=True):
    x = _f32(x)
    if nhwc:
        N, H, W, Cc = x.shape
    else:
        N, Cc, H, W = x.shape
    Ho, Wo = (H + 2 * pad - k) // stride + 1, (W + 2 * pad - k) // stride + 1
    y = np.empty((N, Ho, Wo, Cc) if nhwc else (N, Cc, Ho, Wo), np.float32)
    lib().ref_maxpool(_p(x), _p(y), N, H, W, Cc, k, stride, pad, int(nhwc))
    return y


def avgpool(x, nhwc=True):
    x = _f32(x)
    if nhwc:
        N, HW, Cc = x.shape[0], x.shape[1] * x.shape[2], x.shape[3]
    else:
        N, Cc, HW = x.shape[0], x.shape[1], x.shape[2] * x.shape[3]
    y = np.empty((N, Cc), np.float32)
    lib().ref_avgpool(_p(x), _p(y), N, HW, Cc, int(nhwc))
    return y


def embedding(ids, type_ids, word, pos, typ, seq):
    ids = np.ascontiguousarray(ids, np.int64).ravel()
    tids = None if type_ids is None else np.ascontiguousarray(type_ids, np.int64).ravel()
    word, pos, typ = _f32(word), _f32(pos), _f32(typ)
    width = word.shape[1]
    y = np.empty((ids.size, width), np.float32)
    lib().ref_embedding(_p(ids), _p(tids), _p(word), _p(pos), _p(typ), _p(y), C.c_long(ids.size), seq, width)
    return y
