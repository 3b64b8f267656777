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
