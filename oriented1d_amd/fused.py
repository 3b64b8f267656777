"""Forward-only glue of a ConvNeXt-1D block on the GPU, one pass each, in place of the PyTorch
passes the reference spends around the operator (``models/convnext.py:306-318``: permute +
LayerNorm before the pointwise layers, layer scale + permute + residual after them; the
channels-last LayerNorm + GELU of the stem, ``:176-190``).  The harness uses them when no
gradient is being recorded; with autograd on it composes the same values from PyTorch ops."""
import ctypes

import torch

from . import _lib

_DTYPES = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}
MAX_C_ROWS, MAX_C_TILE = 2048, 1536


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _stream(t):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _f32(p):
    from .dwoconv1d import f32_copy
    return f32_copy(p)


def usable(x, C, tiled):
    """True when the fused kernels cover this call: CUDA tensor of a supported type, even C
    within the kernels' limit, and autograd switched off (they have no backward; with gradients
    enabled the callers compose the same values from PyTorch ops)."""
    return (x.is_cuda and x.dtype in _DTYPES and C % 2 == 0
            and C <= (MAX_C_TILE if tiled else MAX_C_ROWS) and not torch.is_grad_enabled())


def layernorm_nhwc(x, weight, bias, eps, gelu=False):
    """LayerNorm over the last dimension of a contiguous tensor (+ exact GELU)."""
    if not x.is_cuda or x.dtype not in _DTYPES:
        raise RuntimeError("x must be a CUDA tensor of type float32, bfloat16 or float16")
    x = x.contiguous()
    C = x.shape[-1]
    out = torch.empty_like(x)
    g, b = _f32(weight), _f32(bias)  # held until the launch is queued
    _lib.check(_lib.load().dwo_layernorm_nhwc(
        _ptr(x), _ptr(g), _ptr(b), _ptr(out), x.numel() // C, C, float(eps), int(gelu),
        _DTYPES[x.dtype], _stream(x)), "dwo_layernorm_nhwc")
    return out


def nchw_layernorm_nhwc(x, weight, bias, eps):
    """[N,C,H,W] -> [N,H,W,C], LayerNorm over C: ``norm(x.permute(0, 2, 3, 1))`` in one pass."""
    if not x.is_cuda or x.dtype not in _DTYPES:
        raise RuntimeError("x must be a CUDA tensor of type float32, bfloat16 or float16")
    x = x.contiguous()
    N, C, H, W = x.shape
    out = torch.empty((N, H, W, C), dtype=x.dtype, device=x.device)
    g, b = _f32(weight), _f32(bias)
    _lib.check(_lib.load().dwo_nchw_layernorm_nhwc(
        _ptr(x), _ptr(g), _ptr(b), _ptr(out), N, C, H, W, float(eps), _DTYPES[x.dtype],
        _stream(x)), "dwo_nchw_layernorm_nhwc")
    return out


def nhwc_scale_add_nchw(y, scale=None, residual=None):
    """[N,H,W,C] -> [N,C,H,W]: ``residual + (scale * y).permute(0, 3, 1, 2)`` in one pass
    (``scale`` [C] and ``residual`` [N,C,H,W] optional)."""
    if not y.is_cuda or y.dtype not in _DTYPES:
        raise RuntimeError("y must be a CUDA tensor of type float32, bfloat16 or float16")
    y = y.contiguous()
    N, H, W, C = y.shape
    if residual is not None:
        if tuple(residual.shape) != (N, C, H, W) or residual.dtype != y.dtype:
            raise RuntimeError("residual must be [N,C,H,W] of the same type as y")
        residual = residual.contiguous()
    out = torch.empty((N, C, H, W), dtype=y.dtype, device=y.device)
    sc = _f32(scale) if scale is not None else None
    _lib.check(_lib.load().dwo_nhwc_scale_add_nchw(
        _ptr(y), _ptr(sc), _ptr(residual), _ptr(out), N, C, H, W, _DTYPES[y.dtype], _stream(y)),
        "dwo_nhwc_scale_add_nchw")
    return out


def pointwise_dwconv_nhwc(x, linear, conv):
    """``conv(linear(x))`` for a channels-last ``x`` [N,H,W,Cin] (Cin <= 4), an ``nn.Linear``
    Cin -> C and an NHWC ``DepthwiseOrientedConv1d`` over C channels, without writing the
    C-channel tensor (the stem's ``dw1(pw1(x))``, models/convnext.py:177-178)."""
    if not x.is_cuda or x.dtype not in _DTYPES:
        raise RuntimeError("x must be a CUDA tensor of type float32, bfloat16 or float16")
    x = x.contiguous()
    N, H, W, Cin = x.shape
    C, K, stride = conv.out_channels, conv.kernel_size[1], conv.stride[0]
    w = _f32(conv.weight)
    if conv.resid is not None:
        w = w + conv.resid.to(w)
    taps = conv._taps.get(conv.theta, C, K, x.device)  # cached per theta version
    P, Q = -(-H // stride), -(-W // stride)
    y = torch.empty((N, P, Q, C), dtype=x.dtype, device=x.device)
    pw_w = _f32(linear.weight)
    pw_b = _f32(linear.bias) if linear.bias is not None else None
    w2 = w.reshape(C, K)
    cb = _f32(conv.bias) if conv.bias is not None else None
    _lib.check(_lib.ready(x.device).dwo_pointwise_fprop_nhwc(
        _ptr(x), _ptr(pw_w), _ptr(pw_b), _ptr(w2), _ptr(cb), _ptr(taps), _ptr(y), N, Cin, C, H, W,
        K, stride, _DTYPES[x.dtype], _stream(x)), "dwo_pointwise_fprop_nhwc")
    return y
