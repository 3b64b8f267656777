"""GPU checks of the operator module (autograd contract of dwoconv1d.py:18-69)."""
import math

import numpy as np
import pytest
import torch

from parity_util import assert_close, grouped_theta, host

pytestmark = pytest.mark.gpu

from oriented1d_amd import DepthwiseOrientedConv1d  # noqa: E402


def _mk(C, K, stride=1, nhwc=False, resid=False, bias=True, offset=0.0, arbitrary=False):
    m = DepthwiseOrientedConv1d(C, C, K, groups=C, stride=stride, padding=K // 2, bias=bias,
                                angle=[float(t) for t in grouped_theta(C, offset)], nhwc=nhwc,
                                resid=resid, arbitrary_size=arbitrary)
    torch.manual_seed(1)
    torch.nn.init.normal_(m.weight, std=0.02)
    if bias:
        torch.nn.init.normal_(m.bias, std=0.5)
    return m.cuda()


@pytest.mark.parametrize("nhwc", [False, True], ids=["nchw", "nhwc"])
@pytest.mark.parametrize("resid", [False, True], ids=["plain", "resid"])
@pytest.mark.parametrize("stride", [1, 2])
def test_forward_backward_matches_oracle(oracle, nhwc, resid, stride):
    C, K, N, H, W = 48, 15, 2, 16, 20
    m = _mk(C, K, stride, nhwc, resid)
    rng = np.random.default_rng(3)
    x_nchw = rng.standard_normal((N, C, H, W)).astype(np.float32)
    x_np = np.ascontiguousarray(x_nchw.transpose(0, 2, 3, 1)) if nhwc else x_nchw
    x = torch.from_numpy(x_np).cuda().requires_grad_()
    y = m(x)
    w, b, th = host(m.weight), host(m.bias), host(m.theta)
    y_ref = oracle.module_forward(x_np, w, th, bias=b, stride=stride, nhwc=nhwc, resid=resid)
    assert_close(host(y), y_ref, torch.float32, "forward")
    dy_np = rng.standard_normal(y_ref.shape).astype(np.float32)
    y.backward(torch.from_numpy(dy_np).cuda())
    dx, dw, db = oracle.module_backward(dy_np, x_np, w, th, stride=stride, nhwc=nhwc, resid=resid)
    assert_close(host(x.grad), dx, torch.float32, "dx")
    assert_close(host(m.weight.grad), dw, torch.float32, "dw")
    assert_close(host(m.bias.grad), db, torch.float32, "db")
    assert m.theta.grad is None  # dwoconv1d.py:64
    assert m.weight.grad.shape == m.weight.shape and m.weight.grad.dtype == m.weight.dtype


def test_resid_identity_and_needs_input_grad_gating():
    C, K = 32, 31
    m = _mk(C, K, resid=True)
    with torch.no_grad():
        m.weight.zero_()
    x = torch.randn(2, C, 14, 14, device="cuda")
    # w = 0 with the residual tap: y = x + bias exactly
    assert torch.equal(m(x), x + m.bias.view(1, -1, 1, 1))
    # x does not require grad: only parameter grads are produced
    y = m(x)
    y.sum().backward()
    assert m.weight.grad is not None and m.bias.grad is not None
    # frozen weight: dx only
    m2 = _mk(C, K)
    m2.weight.requires_grad_(False)
    m2.bias.requires_grad_(False)
    x2 = x.clone().requires_grad_()
    m2(x2).sum().backward()
    assert x2.grad is not None and m2.weight.grad is None and m2.bias.grad is None


def test_reference_errors_and_arbitrary_size(oracle):
    C, K = 16, 7
    m = _mk(C, K, stride=2)
    with pytest.raises(RuntimeError, match="not divisible by stride"):
        m(torch.randn(1, C, 9, 8, device="cuda"))
    with pytest.raises(RuntimeError, match="unsupported dtype"):
        m(torch.zeros(1, C, 8, 8, device="cuda", dtype=torch.float64))
    ma = _mk(C, K, stride=2, arbitrary=True)
    x = torch.randn(1, C, 9, 11, device="cuda")
    y = ma(x)
    assert tuple(y.shape) == (1, C, 5, 6)
    ref = oracle.module_forward(host(x), host(ma.weight), host(ma.theta), bias=host(ma.bias), stride=2)
    assert_close(host(y), ref, torch.float32, "arbitrary size")
    # non-contiguous input is made contiguous, as the reference does (dwoconv1d.py:24)
    xt = torch.randn(1, 8, 8, C, device="cuda").permute(0, 3, 1, 2)
    assert torch.equal(m(xt), m(xt.contiguous()))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
def test_low_precision_activations_and_autocast(oracle, dtype):
    C, K = 64, 31
    m = _mk(C, K, nhwc=True, resid=True)
    x32 = torch.randn(2, 12, 12, C, device="cuda")
    x = x32.to(dtype).requires_grad_()
    with torch.autocast("cuda", dtype=dtype):
        y = m(x)
    assert y.dtype == dtype
    ref = oracle.module_forward(host(x), host(m.weight), host(m.theta), bias=host(m.bias),
                                nhwc=True, resid=True)
    assert_close(host(y), ref, dtype, "autocast forward")
    y.float().sum().backward()
    assert x.grad.dtype == dtype and m.weight.grad.dtype == torch.float32
    # theta edits are picked up (tap cache is keyed on the parameter version)
    with torch.no_grad():
        m.theta.add_(math.pi / 8)
    ref2 = oracle.module_forward(host(x), host(m.weight), host(m.theta), bias=host(m.bias),
                                 nhwc=True, resid=True)
    assert_close(host(m(x)), ref2, dtype, "after theta edit")


def _tuple_inputs(C, K, N, H, W, stride, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    w = (rng.standard_normal((C, 1, 1, K)) * 0.05).astype(np.float32)
    theta = grouped_theta(C, 0.5)
    dy = rng.standard_normal((N, C, H // stride, W // stride)).astype(np.float32)
    return x, w, theta, dy


@pytest.mark.parametrize("stride", [1, 2])
def test_five_function_tuple_on_gpu(oracle, stride):
    """The reference's boundary (dwoconv1d.py:72-80): fprop(x,w,theta), dgrad(dy,w,theta),
    wgrad(dy,x,theta) and the two transposes of the tuple, each against the oracle."""
    from oriented1d_amd import oriented_dwconv1d_get_module_from_params

    C, K, N, H, W = 40, 15, 2, 16, 24
    x, w, theta, dy = _tuple_inputs(C, K, N, H, W, stride, 7)
    f, d, g, nhwc_to_nchw, nchw_to_nhwc = oriented_dwconv1d_get_module_from_params(
        "float", K, stride, K // 2, Sb=1)
    xd, wd, dyd = (torch.from_numpy(a).cuda() for a in (x, w, dy))
    th = torch.from_numpy(theta).cuda()
    assert_close(host(f(xd, wd, th)), oracle.fprop(x, w, theta, stride), torch.float32, "tuple fprop")
    assert_close(host(d(dyd, wd, th)), oracle.dgrad(dy, w, theta, stride), torch.float32, "tuple dgrad")
    dw = g(dyd, xd, th)
    assert dw.shape == (C, 1, 1, K)
    assert_close(host(dw), oracle.wgrad(dy, x, theta, K, stride), torch.float32, "tuple wgrad")
    # a second call reuses the tuple's cached tap table and gives the same bits
    assert torch.equal(f(xd, wd, th), f(xd, wd, th))
    xn = nchw_to_nhwc(xd)
    assert xn.is_contiguous() and tuple(xn.shape) == (N, H, W, C)
    assert torch.equal(nhwc_to_nchw(xn), xd)
    if stride == 2:
        with pytest.raises(RuntimeError, match="not divisible by stride"):
            f(xd[:, :, :15].contiguous(), wd, th)


@pytest.mark.parametrize("plain", [False, True], ids=["kernel_tuple", "plain_tuple"])
@pytest.mark.parametrize("nhwc", [False, True], ids=["nchw", "nhwc"])
def test_apply_with_the_reference_tuple_in_slot_5(oracle, nhwc, plain):
    """``apply(x, w, theta, bias, module_fp32, nhwc, resid)`` exactly as the reference's forward()
    calls it (dwoconv1d.py:189-198).  A plain 5-tuple of the same functions goes through the
    reference's own composition (transposes, separate bias add, dy.sum)."""
    from oriented1d_amd import _DepthwiseOrientedConv1d, oriented_dwconv1d_get_module_from_params

    C, K, N, H, W = 24, 31, 2, 14, 18
    x, w, theta, dy = _tuple_inputs(C, K, N, H, W, 1, 9)
    rng = np.random.default_rng(10)
    b = rng.standard_normal(C).astype(np.float32)
    resid = np.zeros((C, 1, 1, K), np.float32)
    resid[..., K // 2] = 1
    kt = oriented_dwconv1d_get_module_from_params("float", K, 1, K // 2, Sb=1)
    module = tuple(kt) if plain else kt
    x_np = np.ascontiguousarray(x.transpose(0, 2, 3, 1)) if nhwc else x
    dy_np = np.ascontiguousarray(dy.transpose(0, 2, 3, 1)) if nhwc else dy
    xd = torch.from_numpy(x_np).cuda().requires_grad_()
    wd = torch.from_numpy(w).cuda().requires_grad_()
    bd = torch.from_numpy(b).cuda().requires_grad_()
    th = torch.nn.Parameter(torch.from_numpy(theta).cuda())
    y = _DepthwiseOrientedConv1d.apply(xd, wd, th, bd, module, nhwc, torch.from_numpy(resid).cuda())
    y_ref = oracle.module_forward(x_np, w, theta, bias=b, nhwc=nhwc, resid=True)
    assert_close(host(y), y_ref, torch.float32, "apply forward")
    y.backward(torch.from_numpy(dy_np).cuda())
    dx, dw, db = oracle.module_backward(dy_np, x_np, w, theta, nhwc=nhwc, resid=True)
    assert_close(host(xd.grad), dx, torch.float32, "apply dx")
    assert_close(host(wd.grad), dw, torch.float32, "apply dw")
    assert_close(host(bd.grad), db, torch.float32, "apply db")
    assert th.grad is None


def test_module_attributes_of_the_reference():
    """module_fp32 / module_fp32_large (dwoconv1d.py:144-152) exist, are what forward() passes,
    and survive deepcopy (model averaging copies the model)."""
    import copy

    from oriented1d_amd.dwoconv1d import KernelTuple

    m = _mk(16, 7, stride=2, arbitrary=True)
    assert isinstance(m.module_fp32, tuple) and len(m.module_fp32) == 5
    assert isinstance(m.module_fp32_large, KernelTuple) and m.module_fp32_large.arbitrary_size
    assert not m.module_fp32.arbitrary_size and m.module_fp32.stride == 2
    assert not hasattr(_mk(16, 7), "module_fp32_large")
    m2 = copy.deepcopy(m)
    x = torch.randn(1, 16, 9, 11, device="cuda")
    assert torch.equal(m2(x), m(x))


@pytest.mark.parametrize("stride", [1, 2])
def test_forward_safe_nhwc_odd_sizes(oracle, stride):
    """forward_safe on a channels-last tensor whose extents the stride does not divide
    (dwoconv1d.py:154-187 pads, permutes and crops; the values are those of the cropped result)."""
    C, K = 20, 13
    m = _mk(C, K, stride=stride, nhwc=True, resid=True, arbitrary=True)
    x = torch.randn(2, 17, 23, C, device="cuda", requires_grad=True)
    y = m.forward_safe(x)
    assert tuple(y.shape) == (2, -(-17 // stride), -(-23 // stride), C) and y.is_contiguous()
    args = (host(m.weight), host(m.theta))
    ref = oracle.module_forward(host(x), *args, bias=host(m.bias), stride=stride, nhwc=True, resid=True)
    assert_close(host(y), ref, torch.float32, "forward_safe nhwc")
    assert torch.equal(m(x), y)  # forward is forward_safe for arbitrary_size modules
    dy = torch.randn_like(y)
    y.backward(dy)
    dx, dw, db = oracle.module_backward(host(dy), host(x), *args, stride=stride, nhwc=True, resid=True)
    assert_close(host(x.grad), dx, torch.float32, "forward_safe dx")
    assert_close(host(m.weight.grad), dw, torch.float32, "forward_safe dw")
    assert_close(host(m.bias.grad), db, torch.float32, "forward_safe db")


def test_tap_table_of_another_size_is_rejected():
    from oriented1d_amd import dwoconv1d as op

    taps = op.build_taps(torch.zeros(8), 8, 31).cuda()
    x = torch.randn(1, 16, 8, 8, device="cuda")
    w = torch.randn(16, 1, 1, 31, device="cuda")
    with pytest.raises(RuntimeError, match="tap table does not match"):
        op.fprop(x, w, taps)
