"""Python face of the CPU oracle for the depthwise oriented 1D convolution.

TEST INFRASTRUCTURE ONLY: imported by tests/, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py``.  The shipped package never imports this module and
has no CPU fallback of its own.

Two independent statements of the reference formulation live here:

* ``fprop/dgrad/wgrad`` (+ ``*_f32``) call ``libdwo_oracle.so`` (``dwo_oracle.c``), the C
  restatement of ``models/dwoconv1d_reference/kernels/kernels.cpp:36-52,71-90,111-126``.
* ``brute_*`` are pure-Python triple loops written from the operator's definition, for
  tiny inputs; they share no code with the C file and are used to pin it.

``module_forward`` / ``module_backward`` restate what the autograd Function around the
kernels does (``models/dwoconv1d/dwoconv1d.py:20-69``): residual centre tap, bias add,
NHWC<->NCHW, and the backward tuple (dx, dw, db).
"""
import ctypes
import math
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libdwo_oracle.so")
_lib = None


def build(force=False):
    """Compile dwo_oracle.c with gcc (Makefile beside this file)."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.check_call(["make", "-s", "-C", _HERE])
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.dwo_oracle_max_threads.restype = ctypes.c_int
    return _lib


def max_threads():
    return int(lib().dwo_oracle_max_threads())


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def out_extent(size, stride):
    """P = ceil(H/stride): equals H/stride on the reference's fast path
    (kernels.cu:19-20) and the cropped extent of forward_safe (dwoconv1d.py:183)."""
    return -(-size // stride)


def taps(theta, S, mode=0):
    """(dh, dw) int32 arrays [C, S] -- kernels.cpp:37,43-44."""
    theta = _f32(np.asarray(theta).reshape(-1))
    C = theta.shape[0]
    dh = np.empty((C, S), dtype=np.int32)
    dw = np.empty((C, S), dtype=np.int32)
    lib().dwo_oracle_taps(_ptr(theta), C, S, S // 2, mode, _ptr(dh), _ptr(dw))
    return dh, dw


def _run(name, a, b, theta, out, N, C, H, W, P, Q, S, stride, threads):
    assert S <= 256 and S % 2 == 1
    fn = getattr(lib(), name)
    fn.restype = None
    fn(_ptr(a), _ptr(b), _ptr(theta), _ptr(out), N, C, H, W, P, Q, S, stride, S // 2, threads)
    return out


def fprop(x, w, theta, stride=1, acc="f64", threads=1):
    """y[n,c,p,q] = sum_s x[n,c,p*str+dh(s),q*str+dw(s)] * w[c,s]; x NCHW."""
    x, theta = _f32(x), _f32(np.asarray(theta).reshape(-1))
    N, C, H, W = x.shape
    w = _f32(w).reshape(C, -1)
    S = w.shape[1]
    P, Q = out_extent(H, stride), out_extent(W, stride)
    out = np.empty((N, C, P, Q), dtype=np.float64 if acc == "f64" else np.float32)
    return _run("dwo_oracle_fprop_" + acc, x, w, theta, out, N, C, H, W, P, Q, S, stride, threads)


def dgrad(dy, w, theta, stride=1, in_hw=None, acc="f64", threads=1):
    """dx[n,c,h,w] = sum_s dy[n,c,(h-dh)/str,(w-dw)/str] * w[c,s] where divisible."""
    dy, theta = _f32(dy), _f32(np.asarray(theta).reshape(-1))
    N, C, P, Q = dy.shape
    H, W = in_hw if in_hw is not None else (P * stride, Q * stride)
    assert out_extent(H, stride) == P and out_extent(W, stride) == Q
    w = _f32(w).reshape(C, -1)
    S = w.shape[1]
    out = np.empty((N, C, H, W), dtype=np.float64 if acc == "f64" else np.float32)
    return _run("dwo_oracle_dgrad_" + acc, dy, w, theta, out, N, C, H, W, P, Q, S, stride, threads)


def wgrad(dy, x, theta, S, stride=1, acc="f64", threads=1):
    """dw[c,s] = sum_{n,p,q} x[n,c,p*str+dh,q*str+dw] * dy[n,c,p,q]; returns [C,1,1,S]."""
    dy, x, theta = _f32(dy), _f32(x), _f32(np.asarray(theta).reshape(-1))
    N, C, H, W = x.shape
    P, Q = dy.shape[2], dy.shape[3]
    assert out_extent(H, stride) == P and out_extent(W, stride) == Q
    out = np.empty((C, 1, 1, S), dtype=np.float64 if acc == "f64" else np.float32)
    return _run("dwo_oracle_wgrad_" + acc, dy, x, theta, out, N, C, H, W, P, Q, S, stride, threads)


def bgrad(dy):
    dy = _f32(dy)
    N, C, P, Q = dy.shape
    out = np.empty((C,), dtype=np.float64)
    lib().dwo_oracle_bgrad_f64(_ptr(dy), _ptr(out), N, C, P, Q)
    return out


# ---------------------------------------------------------------------------------------
# The autograd Function around the kernels (dwoconv1d.py:20-69), NCHW or NHWC tensors.
# ---------------------------------------------------------------------------------------
def effective_weight(w, resid):
    """dwoconv1d.py:22-23,136-139: resid adds 1 to the centre tap."""
    w = np.array(w, dtype=np.float32, copy=True)
    if resid:
        w[..., w.shape[-1] // 2] += np.float32(1)
    return w


def module_forward(x, w, theta, bias=None, stride=1, nhwc=False, resid=False, acc="f64"):
    x = np.asarray(x)
    if nhwc:
        x = x.transpose(0, 3, 1, 2)
    y = fprop(x, effective_weight(w, resid), theta, stride, acc=acc)
    if bias is not None:
        y = y + np.asarray(bias, dtype=y.dtype).reshape(1, -1, 1, 1)
    if nhwc:
        y = y.transpose(0, 2, 3, 1)
    return np.ascontiguousarray(y)


def module_backward(dy, x, w, theta, stride=1, nhwc=False, resid=False, with_bias=True, acc="f64"):
    dy, x = np.asarray(dy), np.asarray(x)
    if nhwc:
        dy, x = dy.transpose(0, 3, 1, 2), x.transpose(0, 3, 1, 2)
    S = np.asarray(w).shape[-1]
    dx = dgrad(dy, effective_weight(w, resid), theta, stride, in_hw=x.shape[2:], acc=acc)
    dw = wgrad(dy, x, theta, S, stride, acc=acc)
    db = bgrad(dy) if with_bias else None
    if nhwc:
        dx = np.ascontiguousarray(dx.transpose(0, 2, 3, 1))
    return dx, dw, db


# ---------------------------------------------------------------------------------------
# Pure-Python brute force (tiny inputs only).  Written from the definition:
# offset(s) = trunc(-sin32(theta)*(s-pad)), trunc(cos32(theta)*(s-pad)) in float32.
# ---------------------------------------------------------------------------------------
def brute_taps(theta_c, S):
    pad = S // 2
    t = np.float32(theta_c)
    # libm double sin/cos rounded to float32; for every angle used in tests the table is
    # insensitive to the last ulp (asserted separately against dwo_oracle_taps modes 0/1).
    s32 = np.float32(math.sin(float(t)))
    c32 = np.float32(math.cos(float(t)))
    out = []
    for s in range(S):
        k = np.float32(s - pad)
        out.append((int(math.trunc(float(np.float32(-s32) * k))),
                    int(math.trunc(float(c32 * k)))))
    return out


def brute_fprop(x, w, theta, stride=1):
    x = np.asarray(x, dtype=np.float64)
    N, C, H, W = x.shape
    w = np.asarray(w, dtype=np.float64).reshape(C, -1)
    S = w.shape[1]
    P, Q = out_extent(H, stride), out_extent(W, stride)
    y = np.zeros((N, C, P, Q))
    for c in range(C):
        tp = brute_taps(np.asarray(theta).reshape(-1)[c], S)
        for n in range(N):
            for p in range(P):
                for q in range(Q):
                    for s, (dh, dw) in enumerate(tp):
                        h, ww = p * stride + dh, q * stride + dw
                        if 0 <= h < H and 0 <= ww < W:
                            y[n, c, p, q] += x[n, c, h, ww] * w[c, s]
    return y


def brute_dgrad(dy, w, theta, stride=1, in_hw=None):
    """Adjoint of brute_fprop by scattering (not the reference's gather form)."""
    dy = np.asarray(dy, dtype=np.float64)
    N, C, P, Q = dy.shape
    H, W = in_hw if in_hw is not None else (P * stride, Q * stride)
    w = np.asarray(w, dtype=np.float64).reshape(C, -1)
    S = w.shape[1]
    dx = np.zeros((N, C, H, W))
    for c in range(C):
        tp = brute_taps(np.asarray(theta).reshape(-1)[c], S)
        for n in range(N):
            for p in range(P):
                for q in range(Q):
                    for s, (dh, dw) in enumerate(tp):
                        h, ww = p * stride + dh, q * stride + dw
                        if 0 <= h < H and 0 <= ww < W:
                            dx[n, c, h, ww] += dy[n, c, p, q] * w[c, s]
    return dx


def brute_wgrad(dy, x, theta, S, stride=1):
    dy = np.asarray(dy, dtype=np.float64)
    x = np.asarray(x, dtype=np.float64)
    N, C, H, W = x.shape
    P, Q = dy.shape[2:]
    dwt = np.zeros((C, 1, 1, S))
    for c in range(C):
        tp = brute_taps(np.asarray(theta).reshape(-1)[c], S)
        for n in range(N):
            for p in range(P):
                for q in range(Q):
                    for s, (dh, dw) in enumerate(tp):
                        h, ww = p * stride + dh, q * stride + dw
                        if 0 <= h < H and 0 <= ww < W:
                            dwt[c, 0, 0, s] += x[n, c, h, ww] * dy[n, c, p, q]
    return dwt
