"""CPU-only checks: the C-ABI library loads and exports every symbol the header declares,
argument validation returns the documented status codes before any GPU work, the host tap
table equals the oracle's, and the operator module keeps the reference's contract
(models/dwoconv1d/dwoconv1d.py:92-152)."""
import ctypes
import math
import os
import re

import numpy as np
import pytest
import torch

from oriented1d_amd import _lib
from oriented1d_amd import dwoconv1d as op

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    header = open(os.path.join(ROOT, "include", "dwoconv1d_hip.h")).read()
    declared = set(re.findall(r"\b(dwo_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations parsed"
    for name in sorted(declared):
        assert hasattr(lib, name), "missing export " + name
    assert declared == set(_lib.SIGNATURES), "ctypes table out of step with the header"
    assert lib.dwo_version() >= 100


def test_argument_validation_status_codes():
    lib = _lib.load()
    one = ctypes.c_void_p(16)  # never dereferenced: validation fails first

    def fprop(N=1, C=1, H=4, W=4, K=7, stride=1, dtype=0, layout=0, x=one):
        return lib.dwo_fprop(x, one, None, one, one, N, C, H, W, K, stride, dtype, layout, None)

    assert fprop(x=None) == -1
    assert fprop(N=0) == -2 and fprop(H=0) == -2
    assert fprop(N=1 << 16, C=1 << 10, H=1 << 4, W=1 << 4) == -2  # >= 2^31 elements
    assert fprop(K=8) == -3 and fprop(K=65) == -3 and fprop(K=0) == -3
    assert fprop(stride=3) == -4
    assert fprop(dtype=7) == -5
    assert fprop(layout=2) == -6
    assert lib.dwo_dgrad(None, one, one, one, 1, 1, 4, 4, 7, 1, 0, 0, None) == -1
    need = lib.dwo_wgrad_scratch_bytes(2, 8, 8, 8, 7, 1, 0, 0)
    assert need > 0
    assert lib.dwo_wgrad(one, one, one, one, None, one, need - 1, 2, 8, 8, 8, 7, 1, 0, 0,
                         None) == -7
    assert lib.dwo_wgrad_scratch_bytes(2, 8, 8, 8, 8, 1, 0, 0) == 0
    for code in (0, -1, -2, -3, -4, -5, -6, -7, -8):
        assert lib.dwo_status_string(code)
    assert lib.dwo_taps_bytes(8, 30) == 0
    with pytest.raises(RuntimeError, match="stride must be"):
        _lib.check(-4, "x")


@pytest.mark.parametrize("K", [7, 13, 15, 27, 31, 63])
def test_host_tap_table_equals_oracle(oracle, K):
    rng = np.random.default_rng(K)
    theta = np.concatenate([np.arange(8) * np.float32(math.pi / 8),
                            [np.float32(math.pi * ((n / 8 + 0.5) % 1)) for n in range(8)],
                            rng.uniform(-math.pi, 2 * math.pi, 48)]).astype(np.float32)
    C = len(theta)
    blob = op.build_taps(torch.from_numpy(theta), C, K)
    dh, dw = op.taps_to_numpy(blob, C, K)
    odh, odw = oracle.taps(theta, K)
    assert (dh == odh).all() and (dw == odw).all()


@pytest.mark.parametrize("layout", ["grouped", "roundrobin", "mixed"])
def test_tap_table_channel_order_cycles_through_classes(layout):
    """The blob's channel order is a permutation of the channels in which, while every class
    still has channels left, eight consecutive entries hold the eight orientation classes."""
    from parity_util import canonical_theta, grouped_theta
    C, K = 96, 31
    theta = {"grouped": grouped_theta(C), "roundrobin": canonical_theta(C),
             "mixed": np.concatenate([grouped_theta(64), np.full(32, 0.3, np.float32)])}[layout]
    blob = op.build_taps(torch.from_numpy(theta.astype(np.float32)), C, K).numpy()
    hdr = blob[:32].view(np.int32)
    cls = blob[hdr[5]:hdr[5] + 4 * C].view(np.int32)
    order = blob[hdr[6]:hdr[6] + 4 * C].view(np.int32)
    assert sorted(order.tolist()) == list(range(C))
    if layout != "mixed":
        assert set(cls.tolist()) == set(range(8))
        for i in range(0, C, 8):
            assert sorted(cls[order[i:i + 8]].tolist()) == list(range(8)), i
    else:
        assert (cls[64:] == -1).all()
        first = cls[order[:72]].reshape(8, 9)  # eight full cycles over 8 classes + "other"
        assert all(sorted(r.tolist()) == [-1] + list(range(8)) for r in first)


def test_module_contract():
    C, K = 16, 31
    angles = [math.pi * (c % 8) / 8 for c in range(C)]
    m = op.DepthwiseOrientedConv1d(C, C, K, groups=C, padding=K // 2, angle=angles, resid=True)
    assert isinstance(m, torch.nn.Conv2d)
    assert list(m.state_dict().keys()) == ["weight", "bias", "theta"]
    assert tuple(m.weight.shape) == (C, 1, 1, K) and tuple(m.bias.shape) == (C,)
    assert tuple(m.theta.shape) == (C,) and m.theta.dtype == torch.float32
    assert m.stride == (1, 1) and m.kernel_size == (1, K) and m.nhwc is False
    assert tuple(m.resid.shape) == (C, 1, 1, K) and m.resid.sum() == C
    assert m.resid[:, 0, 0, K // 2].eq(1).all()
    # scalar angle -> [C,1] (dwoconv1d.py:128-129); no resid -> attribute is None
    m2 = op.DepthwiseOrientedConv1d(C, C, 7, groups=C, angle=0.5, bias=False, nhwc=True, stride=2)
    assert tuple(m2.theta.shape) == (C, 1) and m2.resid is None and m2.bias is None
    assert op._DepthwiseOrientedConv1d.__name__ == "_DepthwiseOrientedConv1d"
    with pytest.raises(AssertionError):
        op.DepthwiseOrientedConv1d(C, C, 8, groups=C)  # even kernel
    with pytest.raises(AssertionError):
        op.DepthwiseOrientedConv1d(C, C, 7, groups=1)  # not depthwise
    # reference check order: device first (kernels.cu:11-13)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        m(torch.zeros(1, C, 8, 8))
    import dwoconv1d as alias
    assert alias.DepthwiseOrientedConv1d is op.DepthwiseOrientedConv1d


def test_five_function_tuple_shape():
    t = op.oriented_dwconv1d_get_module_from_params("float", 31, 1, 15, Sb=1)
    assert len(t) == 5 and all(callable(f) for f in t)
    x = torch.arange(24.).reshape(1, 2, 3, 4)
    assert torch.equal(t[3](t[4](x)), x)


def test_oracle_reproduces_golden_fixture(oracle):
    import sys
    sys.path.insert(0, os.path.join(ROOT, "tests", "golden"))
    from make_golden import config1_inputs

    g = np.load(os.path.join(ROOT, "tests", "golden", "config1_samples.npz"))
    x, w, dy, theta = config1_inputs()
    assert abs(x.astype(np.float64).sum() - g["x_sum"]) < 1e-9
    assert abs(w.astype(np.float64).sum() - g["w_sum"]) < 1e-12
    y = oracle.fprop(x, w, theta, threads=4).reshape(-1)[g["idx"]]
    np.testing.assert_array_equal(y, g["y"])
    dw = oracle.wgrad(dy, x, theta, 31, threads=4).reshape(96, 31)
    np.testing.assert_array_equal(dw, g["dw"])


def test_angles_stay_fp32_under_module_casts():
    """Casting the module to a 16-bit type must not round theta: the tap offsets of the rounded
    angles differ from those of the fp32 ones."""
    C, K = 16, 31
    angles = [math.pi * (c % 8) / 8 for c in range(C)]
    m = op.DepthwiseOrientedConv1d(C, C, K, groups=C, padding=K // 2, angle=angles)
    before = m.theta.detach().clone()
    for cast in (lambda mod: mod.bfloat16(), lambda mod: mod.half(), lambda mod: mod.to(torch.float64),
                 lambda mod: mod.float()):
        m = cast(m)
        assert m.theta.dtype == torch.float32 and torch.equal(m.theta.detach(), before)
    assert m.weight.dtype == torch.float32
    assert m.bfloat16().weight.dtype == torch.bfloat16
    rounded_theta = before.to(torch.bfloat16).float()
    dh0, dw0 = op.taps_to_numpy(op.build_taps(before, C, K), C, K)
    dh1, dw1 = op.taps_to_numpy(op.build_taps(rounded_theta, C, K), C, K)
    assert (dh0 != dh1).any() or (dw0 != dw1).any()


def test_backward_without_upstream_gradient_returns_nones():
    """dwoconv1d.py:42-43: an undefined upstream gradient short-circuits to seven Nones (the
    Function does not materialise gradients, :28)."""
    out = op._DepthwiseOrientedConv1d.backward(object(), None)
    assert out == (None,) * 7


def test_specialized_import_name_and_tuple_contract():
    """models/convnext.py:16-23 imports the module under either name; the tuple in slot 5 of
    apply() carries what the native path needs (dwoconv1d.py:72-80,144-152)."""
    import copy
    import pickle

    import dwoconv1d_specialized as spec
    assert spec.DepthwiseOrientedConv1d is op.DepthwiseOrientedConv1d
    m = op.DepthwiseOrientedConv1d(8, 8, 7, groups=8, stride=2, angle=0.3, arbitrary_size=True)
    assert isinstance(m.module_fp32, op.KernelTuple) and len(m.module_fp32) == 5
    assert (m.module_fp32.kernel_size, m.module_fp32.stride, m.module_fp32.arbitrary_size) == (7, 2, False)
    assert m.module_fp32_large.arbitrary_size
    assert m._taps is m.module_fp32_large.taps
    assert not hasattr(op.DepthwiseOrientedConv1d(8, 8, 7, groups=8), "module_fp32_large")
    for twin in (copy.deepcopy(m), pickle.loads(pickle.dumps(m))):
        assert isinstance(twin.module_fp32, op.KernelTuple) and twin.module_fp32 is not m.module_fp32
        assert twin.module_fp32.stride == 2 and twin.module_fp32_large.arbitrary_size
        assert list(twin.state_dict()) == ["weight", "bias", "theta"]
    # CPU tensors are refused by the tuple's functions too (kernels.cu:11-13)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        m.module_fp32[0](torch.zeros(1, 8, 4, 4), m.weight, m.theta)


def test_state_dict_with_16_bit_theta_loads_as_fp32_values():
    """A checkpoint whose theta was saved in a 16-bit type loads into the fp32 parameter: the
    dtype stays fp32, the values are the rounded ones (the information is gone from the file)."""
    C, K = 8, 15
    angles = [math.pi * c / 8 for c in range(C)]
    m = op.DepthwiseOrientedConv1d(C, C, K, groups=C, angle=angles)
    sd = {k: v.clone() for k, v in m.state_dict().items()}
    sd["theta"] = sd["theta"].to(torch.bfloat16)
    m.load_state_dict(sd)
    assert m.theta.dtype == torch.float32
    assert torch.equal(m.theta.detach(), torch.tensor(angles).to(torch.bfloat16).float())
