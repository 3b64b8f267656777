"""dwo_wgrad_static, the wgrad entry point that allocates nothing (its partial sums live in a
static device array of the library), against dwo_wgrad with a caller-allocated scratch: same
kernels, so the results must be equal bit for bit.  Two calls in a row on the shared array, the
second on a smaller input; then further layouts, element types and kernel families."""
import ctypes
import gc

import numpy as np
import pytest
import torch

from parity_util import canonical_theta, grouped_theta

pytestmark = pytest.mark.gpu

from oriented1d_amd import _lib  # noqa: E402
from oriented1d_amd import dwoconv1d as op  # noqa: E402

STATIC_BYTES = 8 << 20  # DWO_STATIC_SCRATCH_BYTES


def _vp(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _both(N, C, H, W, K, stride, dtype, nhwc, theta, seed, with_bias=True):
    """(dw, db) of dwo_wgrad and of dwo_wgrad_static on the same inputs, through the C ABI."""
    lib = _lib.ready(torch.device("cuda:0"))
    g = torch.Generator(device="cuda").manual_seed(seed)
    P, Q = -(-H // stride), -(-W // stride)
    xs, ys = ((N, H, W, C), (N, P, Q, C)) if nhwc else ((N, C, H, W), (N, C, P, Q))
    x = torch.randn(xs, device="cuda", generator=g).to(dtype)
    dy = torch.randn(ys, device="cuda", generator=g).to(dtype)
    taps = op.build_taps(torch.from_numpy(theta), C, K).cuda()
    code = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}[dtype]
    dims = (N, C, H, W, K, stride, code, int(nhwc))
    nbytes = lib.dwo_wgrad_scratch_bytes(*dims)
    assert 0 < nbytes <= STATIC_BYTES
    scratch = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    # every output exists before the call under test: it must not allocate
    dw_a, dw_b = torch.full((C, K), 7.0, device="cuda"), torch.full((C, K), -7.0, device="cuda")
    db_a = torch.full((C,), 7.0, device="cuda") if with_bias else None
    db_b = torch.full((C,), -7.0, device="cuda") if with_bias else None
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # (tensors of earlier tests that sit in reference cycles are released by the collector
    # whenever it happens to run: not between the two readings below)
    gc.collect()
    torch.cuda.synchronize()
    print("wgrad_static case", dims, "seed", seed, flush=True)
    # device-level free memory: sees an allocation by the library itself (hipMalloc inside the
    # .so), which PyTorch's own counter would not; that counter may only go down (a collected
    # tensor), never up
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    _lib.check(lib.dwo_wgrad_static(_vp(dy), _vp(x), _vp(taps), _vp(dw_b), _vp(db_b), *dims, stream),
               "dwo_wgrad_static")
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] >= free_before
    assert torch.cuda.memory_allocated() <= before
    _lib.check(lib.dwo_wgrad(_vp(dy), _vp(x), _vp(taps), _vp(dw_a), _vp(db_a), _vp(scratch), nbytes,
                             *dims, stream), "dwo_wgrad")
    torch.cuda.synchronize()
    return (dw_a, db_a), (dw_b, db_b)


def _equal(pair):
    (dw_a, db_a), (dw_b, db_b) = pair
    assert torch.isfinite(dw_a).all() and torch.equal(dw_a, dw_b)
    if db_a is not None:
        assert torch.equal(db_a, db_b)


def test_two_calls_in_a_row_second_one_smaller():
    # plane kernels with many image groups per channel, then a smaller problem whose partial sums
    # cover only the start of the array the first call filled
    _equal(_both(64, 96, 56, 56, 31, 1, torch.float32, False, canonical_theta(96), 1))
    _equal(_both(5, 40, 28, 28, 31, 1, torch.float32, False, canonical_theta(40), 2))
    # and the first shape again: nothing of the smaller call may leak into it
    _equal(_both(64, 96, 56, 56, 31, 1, torch.float32, False, canonical_theta(96), 3))


@pytest.mark.parametrize("N,C,H,W,K,stride,dtype,nhwc", [
    (16, 192, 28, 28, 31, 1, torch.bfloat16, True),    # NHWC slice kernels
    (3, 38, 61, 35, 31, 2, torch.float16, False),      # NCHW tile kernel, strided
    (2, 36, 70, 90, 15, 1, torch.float32, True),       # NHWC tile kernel
    (2, 5, 33, 17, 7, 1, torch.float32, True),         # lane = channel kernel (C % 4 != 0)
    (1, 8, 40, 37, 63, 1, torch.float32, False),       # generic kernel (K = 63 at fp32)
    (2, 768, 7, 7, 31, 1, torch.float32, False),       # a single image group: no reduction pass
])
def test_kernel_families_share_the_static_scratch(N, C, H, W, K, stride, dtype, nhwc):
    _equal(_both(N, C, H, W, K, stride, dtype, nhwc, grouped_theta(C, 0.5), N + C, with_bias=N % 2 == 0))


def test_sizes_beyond_the_static_scratch_are_refused():
    lib = _lib.ready(torch.device("cuda:0"))
    dims = (64, 4096, 14, 14, 31, 1, 1, 1)  # 4096 channels x 32 image groups: 16 MiB of partial sums
    assert lib.dwo_wgrad_scratch_bytes(*dims) > STATIC_BYTES
    one = torch.zeros(16, device="cuda")
    rc = lib.dwo_wgrad_static(_vp(one), _vp(one), _vp(one), _vp(one), None, *dims, None)
    assert rc == -9 and b"static scratch" in lib.dwo_status_string(rc)
    # argument checks come first, as in dwo_wgrad
    assert lib.dwo_wgrad_static(None, _vp(one), _vp(one), _vp(one), None, 1, 4, 8, 8, 7, 1, 0, 0, None) == -1
    assert lib.dwo_wgrad_static(_vp(one), _vp(one), _vp(one), _vp(one), None, 1, 4, 8, 8, 8, 1, 0, 0, None) == -3
