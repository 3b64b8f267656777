"""Depthwise oriented 1D convolution operator module for MI355X.

Host-side mirror of the reference's operator module (models/dwoconv1d/dwoconv1d.py): same
class names, constructor, parameters (``weight [C,1,1,K]``, ``bias [C]``, ``theta``),
attributes and autograd contract, so ``models/convnext.py:115-127`` can construct it
unchanged.  All arithmetic happens in ``libdwoconv1d_hip.so`` through the C ABI declared
in ``include/dwoconv1d_hip.h``; tensors here only provide device memory and the stream.

Differences from the reference, all supersets:
* bf16/fp16 activations are computed (fp32 accumulate) instead of being reinterpreted as
  float (reference: kernels.cu:25 casts the pointer whatever the dtype).
* ``nhwc=True`` runs NHWC-native kernels; no transposed copies are made
  (reference: dwoconv1d.py:25-26,36-37,50-51,58-59).
* bias add is fused into fprop and the bias gradient into wgrad
  (reference: dwoconv1d.py:34-35,66-67).
* ``arbitrary_size=True`` needs no pad-to-power-of-two / crop round trip
  (reference: dwoconv1d.py:154-187); the kernels take any H, W and give
  ceil(H/stride) x ceil(W/stride) outputs, the same values that path produces.
"""
import ctypes
import weakref

import numpy as np
import torch
import torch.nn as nn

from . import _lib

__all__ = ["DepthwiseOrientedConv1d"]

_DTYPES = {torch.float32: _lib.F32, torch.bfloat16: _lib.BF16, torch.float16: _lib.F16}


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _stream(t):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _check_activation(t, name):
    # models/dwoconv1d/kernels/kernels.cu:11-13,17-18
    if not t.is_cuda:
        raise RuntimeError("%s must be a CUDA tensor" % name)
    if not t.is_contiguous():
        raise RuntimeError("%s must be contiguous" % name)
    if t.dtype not in _DTYPES:
        raise RuntimeError("%s has unsupported dtype %s" % (name, t.dtype))
    if t.dim() != 4:
        raise RuntimeError("%s must be a 4-d tensor" % name)


def build_taps(theta, C, K):
    """Host tap table for ``theta`` ([C] or [C,1] radians) as a uint8 CPU tensor.

    The table is computed by the library on the host in fp32
    (models/dwoconv1d_reference/kernels/kernels.cpp:37,43-44)."""
    lib = _lib.load()
    th = theta.detach().to(device="cpu", dtype=torch.float32).reshape(-1).contiguous()
    if th.numel() != C:
        raise RuntimeError("theta must hold one angle per channel (%d), got %d" % (C, th.numel()))
    blob = torch.empty(lib.dwo_taps_bytes(C, K), dtype=torch.uint8)
    _lib.check(lib.dwo_build_taps(_ptr(th), C, K, _ptr(blob)), "dwo_build_taps")
    return blob


def taps_to_numpy(blob, C, K):
    """(dh, dw) int arrays [C,K] read back from a host tap blob (inspection / tests)."""
    lib = _lib.load()
    dh, dw = np.empty((C, K), np.int32), np.empty((C, K), np.int32)
    a, b = ctypes.c_int(), ctypes.c_int()
    for c in range(C):
        for s in range(K):
            _lib.check(lib.dwo_taps_get(_ptr(blob), c, s, ctypes.byref(a), ctypes.byref(b)),
                       "dwo_taps_get")
            dh[c, s], dw[c, s] = a.value, b.value
    return dh, dw


class _TapCache:
    """Device tap tables, one per (theta tensor, device, C, K), rebuilt when theta is modified
    or moved.  A module owns one (a single entry in practice); the five-function tuple of
    ``oriented_dwconv1d_get_module_from_params`` owns one that may serve several layers, so the
    few most recent tables are kept."""

    KEEP = 8

    def __init__(self):
        self.entries = {}  # (id(theta), device, C, K) -> (state key, weak ref, device blob)

    def get(self, theta, C, K, device):
        slot = (id(theta), str(device), C, K)
        state = (theta.data_ptr(), theta._version)
        hit = self.entries.get(slot)
        if hit is None or hit[0] != state or hit[1]() is not theta:
            if len(self.entries) >= self.KEEP:
                self.entries.pop(next(iter(self.entries)))
            blob = build_taps(theta, C, K).to(device)
            hit = (state, weakref.ref(theta), blob)
            self.entries[slot] = hit
        return hit[2]


def _check_taps(taps, C, K):
    """The device kernels index the tap blob with the C and K they are launched with and cannot
    see its header without a device read, so the size is checked here: a blob of
    ``dwo_taps_bytes(C, K)`` bytes keeps every table read in range."""
    want = _lib.load().dwo_taps_bytes(C, K)
    if taps.dtype != torch.uint8 or taps.numel() != want:
        raise RuntimeError("tap table does not match C=%d, K=%d (%d bytes, expected %d)"
                           % (C, K, taps.numel(), want))


def _dims(x, nhwc):
    if nhwc:
        N, H, W, C = x.shape
    else:
        N, C, H, W = x.shape
    return N, C, H, W


def _out_shape(N, C, H, W, stride, nhwc):
    P, Q = -(-H // stride), -(-W // stride)
    return (N, P, Q, C) if nhwc else (N, C, P, Q)


def _w2d(w, C):
    w = w.detach().reshape(C, -1)
    return w.to(torch.float32).contiguous()


_F32_COPIES = {}  # id(parameter) -> (weak reference, state key, fp32 copy)


def f32_copy(p):
    """fp32 contiguous copy of a parameter, kept until the parameter is modified or moved (the
    library takes weights, biases and norm parameters as fp32; re-casting 16-bit parameters at
    every call costs a kernel launch each)."""
    if p.dtype == torch.float32 and p.is_contiguous():
        return p.detach()
    key = (p._version, p.data_ptr(), p.dtype, str(p.device))
    hit = _F32_COPIES.get(id(p))
    if hit is None or hit[0]() is not p or hit[1] != key:
        pid = id(p)
        ref = weakref.ref(p, lambda _, pid=pid: _F32_COPIES.pop(pid, None))
        hit = (ref, key, p.detach().to(torch.float32).contiguous())
        _F32_COPIES[pid] = hit
    return hit[2]


def fprop(x, w, taps, stride=1, bias=None, nhwc=False):
    """y = fprop(x, w, theta) (+ bias).  x: [N,C,H,W] or [N,H,W,C]; w: [C,1,1,K]."""
    _check_activation(x, "x")
    lib = _lib.ready(x.device)
    N, C, H, W = _dims(x, nhwc)
    w2 = _w2d(w, C)
    K = w2.shape[1]
    _check_taps(taps, C, K)
    b = f32_copy(bias) if bias is not None else None
    y = torch.empty(_out_shape(N, C, H, W, stride, nhwc), dtype=x.dtype, device=x.device)
    _lib.check(_lib.launch(x.device, lib.dwo_fprop, _ptr(x), _ptr(w2), _ptr(b), _ptr(taps), _ptr(y),
                           N, C, H, W, K, stride, _DTYPES[x.dtype], int(nhwc), _stream(x)),
               "dwo_fprop")
    return y


def dgrad(dy, w, taps, in_hw, stride=1, nhwc=False):
    """dx = dgrad(dy, w, theta); ``in_hw`` is the (H, W) of the forward input."""
    _check_activation(dy, "dy")
    lib = _lib.ready(dy.device)
    H, W = in_hw
    N, C, P, Q = _dims(dy, nhwc)
    if (P, Q) != (-(-H // stride), -(-W // stride)):
        raise RuntimeError("dy extent does not match the input extent and stride")
    w2 = _w2d(w, C)
    K = w2.shape[1]
    _check_taps(taps, C, K)
    dx = torch.empty((N, H, W, C) if nhwc else (N, C, H, W), dtype=dy.dtype, device=dy.device)
    _lib.check(_lib.launch(dy.device, lib.dwo_dgrad, _ptr(dy), _ptr(w2), _ptr(taps), _ptr(dx), N, C,
                           H, W, K, stride, _DTYPES[dy.dtype], int(nhwc), _stream(dy)), "dwo_dgrad")
    return dx


def wgrad(dy, x, taps, K, stride=1, nhwc=False, with_bias=False):
    """(dw [C,1,1,K] fp32, db [C] fp32 or None) = wgrad(dy, x, theta)."""
    _check_activation(dy, "dy")
    _check_activation(x, "x")
    lib = _lib.ready(x.device)
    if dy.dtype != x.dtype:
        raise RuntimeError("dy and x must have the same dtype")
    N, C, H, W = _dims(x, nhwc)
    if tuple(dy.shape) != _out_shape(N, C, H, W, stride, nhwc):
        raise RuntimeError("dy extent does not match the input extent and stride")
    _check_taps(taps, C, K)
    dt, lay = _DTYPES[x.dtype], int(nhwc)
    nbytes = lib.dwo_wgrad_scratch_bytes(N, C, H, W, K, stride, dt, lay)
    scratch = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=x.device)
    dw = torch.empty((C, 1, 1, K), dtype=torch.float32, device=x.device)
    db = torch.empty((C,), dtype=torch.float32, device=x.device) if with_bias else None
    _lib.check(_lib.launch(x.device, lib.dwo_wgrad, _ptr(dy), _ptr(x), _ptr(taps), _ptr(dw), _ptr(db),
                           _ptr(scratch), nbytes, N, C, H, W, K, stride, dt, lay, _stream(x)),
               "dwo_wgrad")
    return dw, db


class KernelTuple(tuple):
    """The reference's five-function tuple ``(fprop, dgrad, wgrad, nhwc_to_nchw, nchw_to_nhwc)``
    (models/dwoconv1d/dwoconv1d.py:72-80) plus what the native path needs to run without the
    transposes: kernel size, stride, a tap-table cache, and whether extents that the stride does
    not divide are accepted."""

    def __new__(cls, functions, kernel_size, stride, arbitrary_size):
        self = super().__new__(cls, functions)
        self.kernel_size, self.stride = kernel_size, stride
        self.arbitrary_size = arbitrary_size
        self.taps = _TapCache()
        return self

    def __reduce__(self):
        # copies (copy.deepcopy of a model, e.g. for an averaged twin) and pickles are rebuilt
        # from the parameters; the tap cache starts empty
        return (oriented_dwconv1d_get_module_from_params,
                ("float", self.kernel_size, self.stride, self.kernel_size // 2,
                 4 if self.arbitrary_size else 1))


class _DepthwiseOrientedConv1d(torch.autograd.Function):
    """Autograd contract of models/dwoconv1d/dwoconv1d.py:18-69.

    ``apply(x, w, theta, bias, module, nhwc, resid)``.  ``module`` is what the reference passes
    in this slot, the tuple returned by ``oriented_dwconv1d_get_module_from_params`` (a
    ``KernelTuple`` here): the convolution then runs natively in the tensor's layout with the
    bias fused.  Any other 5-tuple of callables is driven exactly as the reference drives its
    own (transposes, separate bias add, ``dy.sum``), and the owning ``DepthwiseOrientedConv1d``
    is accepted as well.  backward returns (dx, dw, None, db, None, None, None): theta never
    receives a gradient (dwoconv1d.py:64)."""

    @staticmethod
    def forward(ctx, x, w, theta, bias, module, nhwc=False, resid=None):
        ctx.set_materialize_grads(False)
        if isinstance(module, DepthwiseOrientedConv1d):
            module = module.module_fp32_large if module.arbitrary_size else module.module_fp32
        ctx.plain = None
        if not isinstance(module, KernelTuple):
            return _DepthwiseOrientedConv1d._forward_plain(ctx, x, w, theta, bias, module, nhwc,
                                                           resid)
        stride = module.stride
        C = w.shape[0]
        K = w.shape[-1]
        if K != module.kernel_size:
            raise RuntimeError("weight has %d taps, the kernel tuple was made for %d"
                               % (K, module.kernel_size))
        w_eff = f32_copy(w)
        if resid is not None:
            w_eff = w_eff + resid.to(w_eff)
        x = x.contiguous()
        _check_activation(x, "x")
        N, Cx, H, W = _dims(x, nhwc)
        if Cx != C:
            raise RuntimeError("input has %d channels, weight has %d" % (Cx, C))
        if not module.arbitrary_size and (H % stride != 0 or W % stride != 0):
            # models/dwoconv1d/kernels/kernels.cu:20
            raise RuntimeError("Invalid input size: H,W not divisible by stride")
        taps = module.taps.get(theta, C, K, x.device)

        ctx.stride, ctx.nhwc, ctx.K = stride, nhwc, K
        ctx.with_bias = bias is not None
        ctx.w_dtype = w.dtype
        ctx.b_dtype = bias.dtype if bias is not None else None
        ctx.save_for_backward(x, w_eff, taps)
        return fprop(x, w_eff, taps, stride, bias=bias, nhwc=nhwc)

    @staticmethod
    def _forward_plain(ctx, x, w, theta, bias, module, nhwc, resid):
        # models/dwoconv1d/dwoconv1d.py:21-38, for a caller's own five functions
        f, _, _, nhwc_to_nchw, nchw_to_nhwc = module
        if resid is not None:
            w = w + resid
        x = x.contiguous()
        if nhwc:
            x = nhwc_to_nchw(x)
        ctx.plain, ctx.nhwc = module, nhwc
        ctx.save_for_backward(x, w, theta, bias)
        y = f(x, w, theta)
        if bias is not None:
            y = y + bias.to(y).view(1, -1, 1, 1)
        return nchw_to_nhwc(y) if nhwc else y

    @staticmethod
    def backward(ctx, dy):
        if dy is None:
            return None, None, None, None, None, None, None
        if ctx.plain is not None:
            # models/dwoconv1d/dwoconv1d.py:45-69
            _, d, g, nhwc_to_nchw, nchw_to_nhwc = ctx.plain
            x, w, theta, bias = ctx.saved_tensors
            dy = dy.contiguous()
            if ctx.nhwc:
                dy = nhwc_to_nchw(dy)
            dx = dw = db = None
            if ctx.needs_input_grad[0]:
                dx = d(dy, w, theta)
                if ctx.nhwc:
                    dx = nchw_to_nhwc(dx)
            if ctx.needs_input_grad[1]:
                dw = g(dy, x, theta)
            if bias is not None and ctx.needs_input_grad[3]:
                db = dy.sum(dim=[0, 2, 3])
            return dx, dw, None, db, None, None, None
        x, w_eff, taps = ctx.saved_tensors
        dy = dy.contiguous()
        if dy.dtype != x.dtype:
            dy = dy.to(x.dtype)
        N, C, H, W = _dims(x, ctx.nhwc)
        dx = dw = db = None
        if ctx.needs_input_grad[0]:
            dx = dgrad(dy, w_eff, taps, (H, W), ctx.stride, nhwc=ctx.nhwc)
        need_db = ctx.with_bias and ctx.needs_input_grad[3]
        if ctx.needs_input_grad[1]:
            dw, db32 = wgrad(dy, x, taps, ctx.K, ctx.stride, nhwc=ctx.nhwc, with_bias=need_db)
            dw = dw.to(ctx.w_dtype)
            if need_db:
                db = db32.to(ctx.b_dtype)
        elif need_db:
            red = [0, 1, 2] if ctx.nhwc else [0, 2, 3]
            db = dy.sum(dim=red, dtype=torch.float32).to(ctx.b_dtype)
        return dx, dw, None, db, None, None, None


def oriented_dwconv1d_get_module_from_params(ftype, kernel_size, stride, pad, Sb=None):
    """Five-function tuple in the reference's order (models/dwoconv1d/dwoconv1d.py:72-80):
    (fprop(x,w,theta), dgrad(dy,w,theta), wgrad(dy,x,theta), nhwc_to_nchw, nchw_to_nhwc),
    all on contiguous NCHW tensors; the result goes into slot 5 of
    ``_DepthwiseOrientedConv1d.apply`` as in the reference (dwoconv1d.py:189-198).
    ``ftype`` and ``pad`` are accepted for signature compatibility: there is nothing to compile
    per configuration and pad is always ``kernel_size // 2``.  The kernels need no filter
    partitioning; ``Sb=4`` is how the reference asks for its arbitrary-size variant
    (dwoconv1d.py:150-152), so such a tuple accepts extents the stride does not divide
    (output ceil(H/stride)), any other rejects them as kernels.cu:20 does."""
    K = int(kernel_size)
    stride = int(stride)
    arbitrary = Sb is not None and int(Sb) > 1

    def f(x, w, theta):
        if not arbitrary and (x.shape[2] % stride != 0 or x.shape[3] % stride != 0):
            raise RuntimeError("Invalid input size: H,W not divisible by stride")
        return fprop(x, w, kt.taps.get(theta, x.shape[1], K, x.device), stride)

    def d(dy, w, theta):
        hw = (dy.shape[2] * stride, dy.shape[3] * stride)
        return dgrad(dy, w, kt.taps.get(theta, dy.shape[1], K, dy.device), hw, stride)

    def g(dy, x, theta):
        return wgrad(dy, x, kt.taps.get(theta, x.shape[1], K, x.device), K, stride)[0].to(x.dtype)

    def nhwc_to_nchw(x):
        return x.permute(0, 3, 1, 2).contiguous()

    def nchw_to_nhwc(x):
        return x.permute(0, 2, 3, 1).contiguous()

    kt = KernelTuple((f, d, g, nhwc_to_nchw, nchw_to_nhwc), K, stride, arbitrary)
    return kt


class DepthwiseOrientedConv1d(nn.Conv2d):
    """Drop-in for models/dwoconv1d/dwoconv1d.py:92-198.

    ``padding`` only shapes the parent ``nn.Conv2d``; the compute path always pads by
    ``kernel_size // 2`` (dwoconv1d.py:133)."""

    def __init__(
        self,
        in_channels,
        out_channels,
        kernel_size=3,
        *,
        groups=1,
        stride=1,
        padding=1,
        bias=True,
        angle=0,
        nhwc=False,
        resid=False,
        arbitrary_size=False,
    ):
        super().__init__(
            in_channels,
            out_channels,
            (1, kernel_size),
            groups=groups,
            stride=stride,
            padding=(0, padding),
            bias=bias,
        )
        assert (
            isinstance(kernel_size, int)
            and in_channels == out_channels
            and groups == in_channels
            and kernel_size % 2 == 1
        )
        assert self.stride[0] == self.stride[1]
        assert kernel_size <= 63 and self.stride[0] in (1, 2, 4)

        if isinstance(angle, (float, int)):
            angle = torch.zeros((in_channels, 1)) + angle
        self.theta = nn.Parameter(torch.as_tensor(angle, dtype=torch.float32).clone(),
                                  requires_grad=True)
        self.nhwc = nhwc
        self.arbitrary_size = arbitrary_size
        pad = kernel_size // 2
        if resid:
            onehot = torch.zeros_like(self.weight.detach())
            onehot[:, :, :, pad:pad + 1] = 1
            # follows .to()/.cuda() with the module, not part of the state_dict
            self.register_buffer("resid", onehot, persistent=False)
        else:
            self.resid = None
        # models/dwoconv1d/dwoconv1d.py:144-152: the tuples forward() hands to apply()
        self.module_fp32 = oriented_dwconv1d_get_module_from_params(
            "float", kernel_size, self.stride[0], pad, Sb=1)
        if arbitrary_size:
            self.module_fp32_large = oriented_dwconv1d_get_module_from_params(
                "float", kernel_size, self.stride[0], pad, Sb=4)

    def _apply(self, fn, recurse=True):
        """``.to()/.half()/.bfloat16()/.cuda()`` move and cast weight and bias, but the angles stay
        fp32: they are geometry, and their tap offsets (``(int)(cosf(theta) * k)``) change when
        theta is rounded to a 16-bit type (the reference supports fp32 only and would
        reinterpret the bits, kernels.cu:25)."""
        theta = self.theta.data
        super()._apply(fn, recurse)
        if self.theta.dtype != torch.float32:
            self.theta.data = theta.to(self.theta.device)
        return self

    @property
    def _taps(self):
        """Tap-table cache of the tuple forward() uses."""
        return (self.module_fp32_large if self.arbitrary_size else self.module_fp32).taps

    def forward_safe(self, x):
        """Arbitrary H, W (reference: dwoconv1d.py:154-187): no padding to a power of two, no
        crop and no permuted copies; the kernels produce ceil(H/stride) x ceil(W/stride)
        outputs in the tensor's own layout, the values that path returns."""
        return _DepthwiseOrientedConv1d.apply(
            x, self.weight, self.theta, self.bias, self.module_fp32_large, self.nhwc, self.resid
        )

    def forward(self, x):
        if self.arbitrary_size:  # the reference rebinds forward to forward_safe (:148-149)
            return self.forward_safe(x)
        return _DepthwiseOrientedConv1d.apply(
            x, self.weight, self.theta, self.bias, self.module_fp32, self.nhwc, self.resid
        )
