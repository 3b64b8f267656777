"""Helpers shared by the GPU parity tests."""
import math

import numpy as np
import torch

# north-star tolerances: fp32 within 1e-5 relative, bf16/fp16 (fp32 accumulate) within 1e-2
TOL = {torch.float32: 1e-5, torch.bfloat16: 1e-2, torch.float16: 1e-2}


def canonical_theta(C):
    """theta_c = (c mod 8) * 22.5 degrees, round-robin (benchmark configurations)."""
    return np.array([(c % 8) * math.pi / 8 for c in range(C)], dtype=np.float32)


def grouped_theta(C, layer_offset=0.0, n_dir=8):
    """Contiguous groups of ~C/8 channels per direction (models/convnext.py:60-77,111-114)."""
    return np.array([math.pi * ((((n_dir * (c + 1) - 1) // C) / n_dir + layer_offset) % 1)
                     for c in range(C)], dtype=np.float32)


def rel_err(got, ref):
    """Tensor-level relative errors: (max|d| / max|ref|, ||d||_2 / ||ref||_2)."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    d = np.abs(got - ref)
    scale = max(np.abs(ref).max(), 1e-30)
    return d.max() / scale, math.sqrt((d ** 2).sum() / max((ref ** 2).sum(), 1e-300))


def assert_close(got, ref, dtype, what=""):
    tol = TOL[dtype]
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    assert np.isfinite(np.asarray(got, dtype=np.float64)).all(), what + ": non-finite output"
    emax, el2 = rel_err(got, ref)
    assert emax <= tol and el2 <= tol, "%s: max-rel %.3e l2-rel %.3e > %.0e" % (what, emax, el2, tol)


def rounded(a, dtype):
    """Round a float32 numpy array through `dtype` (what the GPU sees), back as float32."""
    return torch.from_numpy(np.ascontiguousarray(a)).to(dtype).to(torch.float32).numpy()


def dev(a, dtype):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device="cuda", dtype=dtype)


def host(t):
    return t.detach().to(torch.float32).cpu().numpy()
