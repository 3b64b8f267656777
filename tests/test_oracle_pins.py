"""Pins the CPU oracle (oracle/dwo_oracle.c) without the reference's code.

The reference holds no golden vectors for this path, so the oracle is pinned by what
the mathematics fixes: tap-table known answers, library conv2d closed forms, impulse
responses, adjoint identities and an independent pure-Python brute force.  Each check
is chosen so that a plausible slip (floor instead of truncation, a flipped sign of sin,
correlation vs convolution, a swapped h/w, a wrong stride rule) fails at least one.
"""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

PI8 = [np.float32(k * math.pi / 8) for k in range(8)]


def dense_kernel(theta, w, S):
    """Scatter the S taps of every channel into a (2pad+1)^2 depthwise kernel."""
    from oracle.dwo_oracle import brute_taps

    pad = S // 2
    C = len(theta)
    k2 = torch.zeros(C, 1, 2 * pad + 1, 2 * pad + 1, dtype=torch.float64)
    idx = []
    for c in range(C):
        tp = brute_taps(theta[c], S)
        idx.append(tp)
        for s, (dh, dw) in enumerate(tp):
            k2[c, 0, dh + pad, dw + pad] += float(w[c, s])
    return k2, idx


# ------------------------------------------------------------------ tap-table KATs
def test_taps_known_answers(oracle):
    dh, dw = oracle.taps(PI8, 31)
    distinct = [len({(int(a), int(b)) for a, b in zip(dh[c], dw[c])}) for c in range(8)]
    assert distinct == [31, 29, 21, 29, 31, 29, 21, 29]
    k = np.arange(31) - 15
    # 0 deg: pure horizontal line, dw = s - pad
    assert (dh[0] == 0).all() and (dw[0] == k).all()
    # 90 deg: cos(fp32(pi/2)) = -4.37e-8 -> trunc gives 0 (floor would give -1 for k>0)
    assert (dw[4] == 0).all() and (dh[4] == -k).all()
    # 45 deg: offsets (-d, d), d = trunc(0.70710677*k) in [-10, 10]
    d = np.trunc(np.float32(0.70710677) * k.astype(np.float32)).astype(int)
    assert (dw[2] == d).all() and (dh[2] == -d).all() and d.min() == -10 and d.max() == 10
    # 135 deg: both offsets move together: (-d, -d)
    assert (dw[6] == -d).all() and (dh[6] == -d).all()
    # 22.5 deg: hand-derived sequence (trunc toward zero gives the triple 0 around the centre)
    exp_dw = [-13, -12, -12, -11, -10, -9, -8, -7, -6, -5, -4, -3, -2, -1, 0, 0, 0,
              1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 12, 13]
    assert dw[1].tolist() == exp_dw
    assert dh[1].min() == -5 and dh[1].max() == 5
    # sign convention: positive tap index moves *up* (negative dh) for 0 < theta < 90 deg
    assert dh[1][30] == -5 and dh[1][0] == 5
    # centre tap is always the pixel itself
    assert (dh[:, 15] == 0).all() and (dw[:, 15] == 0).all()


def test_taps_point_symmetry_and_python_twin(oracle):
    from oracle.dwo_oracle import brute_taps

    rng = np.random.default_rng(1)
    theta = np.concatenate([np.array(PI8), rng.uniform(0, math.pi, 24).astype(np.float32)])
    for S in (7, 15, 31):
        dh, dw = oracle.taps(theta, S)
        # truncation is odd-symmetric: offset(-k) = -offset(k)
        assert (dh == -dh[:, ::-1]).all() and (dw == -dw[:, ::-1]).all()
        for c in range(len(theta)):
            assert brute_taps(theta[c], S) == list(zip(dh[c].tolist(), dw[c].tolist()))


def test_taps_insensitive_to_libm_flavour(oracle):
    """sinf/cosf vs double sin/cos rounded to float: same table on every angle the
    workloads use (k*pi/8, and the model's pi*((n/8 + j/2) mod 1))."""
    angles = list(PI8) + [np.float32(math.pi * ((n / 8 + 0.5) % 1)) for n in range(8)]
    for S in (7, 13, 15, 27, 31):
        a = oracle.taps(angles, S, mode=0)
        b = oracle.taps(angles, S, mode=1)
        assert (a[0] == b[0]).all() and (a[1] == b[1]).all()


# ------------------------------------------------------------------ closed forms
def _rand(shape, seed, scale=1.0):
    return (np.random.default_rng(seed).standard_normal(shape) * scale).astype(np.float32)


@pytest.mark.parametrize("stride", [1, 2])
@pytest.mark.parametrize("HW", [(10, 12), (7, 7), (9, 5)])
def test_theta0_is_horizontal_conv2d(oracle, HW, stride):
    N, C, S = 2, 3, 31 if HW == (7, 7) else 7
    x, w = _rand((N, C) + HW, 0), _rand((C, 1, 1, S), 1)
    ref = F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(),
                   padding=(0, S // 2), stride=stride, groups=C).numpy()
    got = oracle.fprop(x, w, np.zeros(C, np.float32), stride)
    assert got.shape == ref.shape
    np.testing.assert_allclose(got, ref, rtol=0, atol=1e-12)


@pytest.mark.parametrize("stride", [1, 2])
def test_theta90_is_flipped_vertical_conv2d(oracle, stride):
    N, C, H, W, S = 2, 3, 12, 8, 7
    x, w = _rand((N, C, H, W), 2), _rand((C, 1, 1, S), 3)
    wv = torch.from_numpy(w).double().flip(-1).view(C, 1, S, 1)
    ref = F.conv2d(torch.from_numpy(x).double(), wv, padding=(S // 2, 0), stride=stride,
                   groups=C).numpy()
    got = oracle.fprop(x, w, np.full(C, np.float32(math.pi / 2)), stride)
    np.testing.assert_allclose(got, ref, rtol=0, atol=1e-12)


@pytest.mark.parametrize("stride,HW", [(1, (10, 12)), (1, (7, 7)), (2, (12, 8)), (2, (9, 11)),
                                       (4, (16, 12)), (4, (13, 18))])
def test_any_theta_matches_dense_2d_kernel_and_its_autograd(oracle, stride, HW):
    """fprop == conv2d with the taps scattered into a dense 2-D kernel; autograd of that
    library op pins dgrad and wgrad (incl. duplicate taps and the ceil(H/stride) extent)."""
    rng = np.random.default_rng(5)
    theta = np.concatenate([np.array(PI8), rng.uniform(0, math.pi, 4).astype(np.float32)])
    N, C, S = 2, len(theta), 31 if HW == (7, 7) else 9
    pad = S // 2
    x, w = _rand((N, C) + HW, 6), _rand((C, S), 7)
    k2, idx = dense_kernel(theta, w, S)
    xt = torch.from_numpy(x).double().requires_grad_()
    k2.requires_grad_()
    yt = F.conv2d(xt, k2, padding=pad, stride=stride, groups=C)
    y = oracle.fprop(x, w, theta, stride)
    assert y.shape == tuple(yt.shape)
    np.testing.assert_allclose(y, yt.detach().numpy(), rtol=0, atol=1e-12)
    dy = _rand(tuple(yt.shape), 8)
    yt.backward(torch.from_numpy(dy).double())
    dx = oracle.dgrad(dy, w, theta, stride, in_hw=HW)
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=0, atol=1e-12)
    dw = oracle.wgrad(dy, x, theta, S, stride)
    exp = np.array([[k2.grad[c, 0, dh + pad, dw_ + pad].item() for dh, dw_ in idx[c]]
                    for c in range(C)])
    np.testing.assert_allclose(dw.reshape(C, S), exp, rtol=0, atol=1e-11)


def test_impulse_response(oracle):
    """x = delta(h0,w0): y[h0-dh(s), w0-dw(s)] accumulates w[s] (duplicates add up)."""
    S, H, W = 31, 33, 35
    C = 8
    x = np.zeros((1, C, H, W), np.float32)
    x[:, :, 16, 17] = 1
    w = _rand((C, S), 11)
    y = oracle.fprop(x, w, PI8)
    dh, dw = oracle.taps(PI8, S)
    exp = np.zeros((C, H, W))
    for c in range(C):
        for s in range(S):
            exp[c, 16 - dh[c, s], 17 - dw[c, s]] += np.float64(w[c, s])
    np.testing.assert_allclose(y[0], exp, rtol=0, atol=1e-12)


@pytest.mark.parametrize("stride", [1, 2, 4])
def test_adjoint_identities(oracle, stride):
    """<fprop(x),dy> = <x,dgrad(dy)> = <w,wgrad(dy,x)>."""
    rng = np.random.default_rng(3)
    theta = rng.uniform(0, math.pi, 6).astype(np.float32)
    N, C, H, W, S = 3, 6, 12, 10, 15
    x, w = _rand((N, C, H, W), 20), _rand((C, S), 21)
    y = oracle.fprop(x, w, theta, stride)
    dy = _rand(y.shape, 22)
    a = (y * dy).sum()
    b = (x.astype(np.float64) * oracle.dgrad(dy, w, theta, stride, in_hw=(H, W))).sum()
    c = (w.astype(np.float64) * oracle.wgrad(dy, x, theta, S, stride).reshape(C, S)).sum()
    assert abs(a - b) < 1e-9 * max(1, abs(a)) and abs(a - c) < 1e-9 * max(1, abs(a))


def test_stride_subsamples_stride1(oracle):
    theta = np.array(PI8)
    x, w = _rand((2, 8, 12, 16), 30), _rand((8, 15), 31)
    y1 = oracle.fprop(x, w, theta, 1)
    for stride in (2, 4):
        np.testing.assert_array_equal(oracle.fprop(x, w, theta, stride), y1[..., ::stride, ::stride])


@pytest.mark.parametrize("stride,HW", [(1, (6, 7)), (2, (6, 8)), (2, (5, 7)), (4, (8, 8)), (4, (9, 6))])
def test_c_oracle_equals_python_brute_force(oracle, stride, HW):
    rng = np.random.default_rng(9)
    theta = np.concatenate([np.array(PI8[1:4]), rng.uniform(0, math.pi, 2).astype(np.float32)])
    N, C, S = 2, len(theta), 9
    x, w = _rand((N, C) + HW, 40), _rand((C, S), 41)
    y = oracle.fprop(x, w, theta, stride)
    np.testing.assert_allclose(y, oracle.brute_fprop(x, w, theta, stride), rtol=0, atol=1e-12)
    dy = _rand(y.shape, 42)
    np.testing.assert_allclose(oracle.dgrad(dy, w, theta, stride, in_hw=HW),
                               oracle.brute_dgrad(dy, w, theta, stride, in_hw=HW), rtol=0, atol=1e-12)
    np.testing.assert_allclose(oracle.wgrad(dy, x, theta, S, stride),
                               oracle.brute_wgrad(dy, x, theta, S, stride), rtol=0, atol=1e-11)


def test_f32_accumulating_variant_and_threads(oracle):
    theta = np.array(PI8)
    x, w = _rand((2, 8, 14, 14), 50), _rand((8, 31), 51, 0.02)
    y64 = oracle.fprop(x, w, theta)
    y32 = oracle.fprop(x, w, theta, acc="f32")
    assert y32.dtype == np.float32
    np.testing.assert_allclose(y32, y64, rtol=1e-5, atol=1e-6)
    # the OpenMP path partitions channels only: bit-identical to one thread
    np.testing.assert_array_equal(oracle.fprop(x, w, theta, acc="f32", threads=4), y32)
    dy = _rand(y64.shape, 52)
    np.testing.assert_array_equal(oracle.wgrad(dy, x, theta, 31, acc="f32", threads=4),
                                  oracle.wgrad(dy, x, theta, 31, acc="f32"))
    np.testing.assert_allclose(oracle.dgrad(dy, w, theta, acc="f32"), oracle.dgrad(dy, w, theta),
                               rtol=1e-5, atol=1e-6)


def test_module_semantics_resid_bias_nhwc(oracle):
    """dwoconv1d.py:20-38: w=0 with resid gives identity (+bias); nhwc == permute.op.permute."""
    theta = np.array(PI8)
    x = _rand((2, 8, 9, 11), 60)
    bias = _rand((8,), 61)
    y = oracle.module_forward(x, np.zeros((8, 1, 1, 7), np.float32), theta, bias=bias, resid=True)
    np.testing.assert_allclose(y, x.astype(np.float64) + bias.reshape(1, -1, 1, 1), atol=1e-12)
    w = _rand((8, 1, 1, 7), 62)
    a = oracle.module_forward(x, w, theta, bias=bias)
    b = oracle.module_forward(np.ascontiguousarray(x.transpose(0, 2, 3, 1)), w, theta, bias=bias,
                              nhwc=True)
    np.testing.assert_array_equal(a, b.transpose(0, 3, 1, 2))
    dy = _rand(a.shape, 63)
    dx, dw, db = oracle.module_backward(dy, x, w, theta)
    np.testing.assert_allclose(db, dy.astype(np.float64).sum((0, 2, 3)), atol=1e-10)
    dx2, dw2, _ = oracle.module_backward(np.ascontiguousarray(dy.transpose(0, 2, 3, 1)),
                                         np.ascontiguousarray(x.transpose(0, 2, 3, 1)), w, theta,
                                         nhwc=True)
    np.testing.assert_array_equal(dx, dx2.transpose(0, 3, 1, 2))
    np.testing.assert_array_equal(dw, dw2)
