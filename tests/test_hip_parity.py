"""GPU parity: the HIP kernels, called through the C ABI, against the CPU oracle on the same
seeded inputs.  Tolerances: fp32 1e-5 relative, bf16/fp16 1e-2 relative (tensor-level, see
parity_util.rel_err); wgrad is judged against the double-accumulating oracle because the
reference's own serial fp32 sum over N*P*Q terms is noisier than 1e-5."""
import math
import os
import sys

import numpy as np
import pytest
import torch

from parity_util import (TOL, assert_close, canonical_theta, dev, grouped_theta, host, rel_err,
                         rounded)

pytestmark = pytest.mark.gpu

from oriented1d_amd import dwoconv1d as op  # noqa: E402

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = [torch.float32, torch.bfloat16, torch.float16]


def _case(oracle, N, C, H, W, K, stride, dtype, nhwc, theta, seed, bias=True, threads=8):
    """Runs fprop, dgrad, wgrad(+db) through the C ABI and checks each against the oracle."""
    rng = np.random.default_rng(seed)
    x = rounded(rng.standard_normal((N, C, H, W)).astype(np.float32), dtype)
    w = (rng.standard_normal((C, 1, 1, K)) * 0.02).astype(np.float32)
    b = rng.standard_normal(C).astype(np.float32) if bias else None
    P, Q = -(-H // stride), -(-W // stride)
    dy = rounded(rng.standard_normal((N, C, P, Q)).astype(np.float32), dtype)
    tag = "N%d C%d %dx%d K%d s%d %s %s" % (N, C, H, W, K, stride, dtype, "nhwc" if nhwc else "nchw")
    print("case", tag, "seed", seed, flush=True)

    def lay(a):
        return np.ascontiguousarray(a.transpose(0, 2, 3, 1)) if nhwc else a

    def unlay(a):
        return a.transpose(0, 3, 1, 2) if nhwc else a

    taps = op.build_taps(torch.from_numpy(theta), C, K).cuda()
    xd, dyd, wd = dev(lay(x), dtype), dev(lay(dy), dtype), dev(w, torch.float32)
    bd = dev(b, torch.float32) if bias else None

    y = unlay(host(op.fprop(xd, wd, taps, stride, bias=bd, nhwc=nhwc)))
    y_ref = oracle.fprop(x, w, theta, stride, threads=threads)
    if bias:
        y_ref = y_ref + b.astype(np.float64).reshape(1, -1, 1, 1)
    assert_close(y, y_ref, dtype, tag + " fprop")

    dx = unlay(host(op.dgrad(dyd, wd, taps, (H, W), stride, nhwc=nhwc)))
    assert_close(dx, oracle.dgrad(dy, w, theta, stride, in_hw=(H, W), threads=threads), dtype,
                 tag + " dgrad")

    dw, db = op.wgrad(dyd, xd, taps, K, stride, nhwc=nhwc, with_bias=True)
    # dw/db are fp32 sums of exact products of the (already rounded) inputs: fp32 tolerance
    assert_close(host(dw), oracle.wgrad(dy, x, theta, K, stride, threads=threads), torch.float32,
                 tag + " wgrad")
    assert_close(host(db), oracle.bgrad(dy), torch.float32, tag + " bgrad")
    torch.cuda.synchronize()


def test_config1_cpu_runnable_case_and_golden(oracle):
    """N=2, C=96, 56x56, K=31, theta=(c mod 8)*22.5deg, seed 0, fp32: full-tensor parity with
    the oracle and with the committed golden samples."""
    sys.path.insert(0, os.path.join(ROOT, "tests", "golden"))
    from make_golden import config1_inputs

    x, w, dy, theta = config1_inputs()
    g = np.load(os.path.join(ROOT, "tests", "golden", "config1_samples.npz"))
    taps = op.build_taps(torch.from_numpy(theta), 96, 31).cuda()
    xd, wd, dyd = dev(x, torch.float32), dev(w, torch.float32), dev(dy, torch.float32)
    y = host(op.fprop(xd, wd, taps))
    assert_close(y, oracle.fprop(x, w, theta, threads=8), torch.float32, "config1 fprop")
    assert_close(y.reshape(-1)[g["idx"]], g["y"], torch.float32, "config1 fprop golden")
    dx = host(op.dgrad(dyd, wd, taps, (56, 56)))
    assert_close(dx.reshape(-1)[g["idx"]], g["dx"], torch.float32, "config1 dgrad golden")
    dw, _ = op.wgrad(dyd, xd, taps, 31)
    assert_close(host(dw).reshape(96, 31), g["dw"], torch.float32, "config1 wgrad golden")


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("nhwc", [False, True], ids=["nchw", "nhwc"])
@pytest.mark.parametrize("C,HW", [(96, 56), (192, 28), (384, 14), (768, 7)])
def test_stage_shapes_k31(oracle, C, HW, nhwc, dtype):
    """ConvNeXt-T stage shapes (batch reduced to 4 so the oracle takes seconds)."""
    _case(oracle, 4, C, HW, HW, 31, 1, dtype, nhwc, canonical_theta(C), seed=C + HW)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("nhwc", [False, True], ids=["nchw", "nhwc"])
@pytest.mark.parametrize("C,HW", [(64, 56), (128, 28), (256, 14), (512, 7)])
def test_stage_shapes_k15(oracle, C, HW, nhwc, dtype):
    """First convolution of the 1D++ blocks: K = 15 at the stage extents, contiguous-group
    angles with the +90 degree offset of odd layers."""
    _case(oracle, 3, C, HW, HW, 15, 1, dtype, nhwc, grouped_theta(C, 0.5), seed=C + HW + 15)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("nhwc", [False, True], ids=["nchw", "nhwc"])
@pytest.mark.parametrize("HW", [56, 28, 14])
def test_reference_benchmark_shapes_k7(oracle, HW, nhwc, dtype):
    """K = 7 at the extents of the reference's own micro-benchmark (analysis/benchmark.py:84-104):
    the eight orientations, and the angles that script really passes (degrees read as radians)."""
    _case(oracle, 3, 64, HW, HW, 7, 1, dtype, nhwc, canonical_theta(64), seed=HW + 7)
    published = np.array([0, 22.5, 45, 66.75, 90, 112.5, 135, 157.5] * 2, dtype=np.float32)
    _case(oracle, 2, 16, HW, HW, 7, 1, dtype, nhwc, published, seed=HW + 8)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("nhwc", [False, True], ids=["nchw", "nhwc"])
@pytest.mark.parametrize("C,HW", [(48, 56), (64, 28), (96, 14), (128, 7)])
def test_stage_shapes_reversed_orientations(oracle, C, HW, nhwc, dtype):
    """Angles of the layers turned by 90 degrees (models/convnext.py:159-160): half of them lie
    in [180, 270) degrees, where the taps are a canonical pattern in reverse order."""
    theta = (canonical_theta(C) + np.float32(math.pi / 2)).astype(np.float32)
    _case(oracle, 3, C, HW, HW, 31, 1, dtype, nhwc, theta, seed=C + HW + 90)
    theta = (canonical_theta(C) + np.float32(math.pi)).astype(np.float32)
    _case(oracle, 2, C, HW, HW, 31, 1, dtype, nhwc, theta, seed=C + HW + 180)


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("C,HW", [(24, 64), (40, 32), (72, 16)])
def test_stage_extents_of_a_512_input(oracle, C, HW, dtype):
    """The stage extents of a 512 x 512 input that have compile-time planes (NCHW): canonical
    angles round-robin and in groups, arbitrary angles mixed in, odd batch sizes that leave
    partial batches and image groups; NHWC at the same extents (tile kernels)."""
    rng = np.random.default_rng(HW)
    _case(oracle, 9, C, HW, HW, 31, 1, dtype, False, canonical_theta(C), seed=HW * 7)
    theta = grouped_theta(C, 0.5)
    theta[2::5] = rng.uniform(-math.pi, 2 * math.pi, len(theta[2::5])).astype(np.float32)
    _case(oracle, 5, C, HW, HW, 31, 1, dtype, False, theta, seed=HW * 7 + 1)
    _case(oracle, 2, C, HW, HW, 31, 1, dtype, True, canonical_theta(C), seed=HW * 7 + 2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("C,HW", [(40, 56), (40, 28), (72, 14), (100, 7)])
def test_stage_shapes_mixed_angles(oracle, C, HW, dtype):
    """Stage plane extents with arbitrary angles mixed among canonical ones (a workgroup picks
    the compile-time or the table-driven body per channel), odd batch and channel counts."""
    rng = np.random.default_rng(HW)
    theta = canonical_theta(C)
    theta[1::3] = rng.uniform(-math.pi, 2 * math.pi, len(theta[1::3])).astype(np.float32)
    _case(oracle, 5, C, HW, HW, 31, 1, dtype, False, theta, seed=HW * 3)
    _case(oracle, 3, C, HW, HW, 31, 1, dtype, False, grouped_theta(C, 0.5), seed=HW * 5)


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("K,HW", [(31, 56), (31, 28), (31, 14), (31, 7), (15, 56), (15, 14), (15, 7),
                                  (7, 28), (7, 14)])
def test_arbitrary_angles_on_every_channel(oracle, K, HW, dtype):
    """Every channel on the table-driven bodies (no canonical angle among them): planes larger
    than K / 2 in both directions, planes that some taps miss altogether (14 x 14 at K = 31,
    7 x 7 at K = 15: angles next to 90 and 0 degrees are among the channels), and 7 x 7 at
    K = 31, where the bodies loop over the live taps; batch sizes that leave partial batches,
    angles on both sides of 180 degrees."""
    rng = np.random.default_rng(K * 100 + HW)
    theta = rng.uniform(-math.pi, 2 * math.pi, 11).astype(np.float32)
    theta[:4] = np.float32([1.55, 1.62, 0.03, 3.1])  # steepest and flattest lines: the far taps leave a small plane
    _case(oracle, 5, 11, HW, HW, K, 1, dtype, False, theta, seed=K + HW)
    _case(oracle, 1, 11, HW, HW, K, 1, dtype, False, theta[::-1].copy(), seed=K + HW + 1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("C,HW", [(64, 14), (96, 7), (72, 14), (40, 7)])
def test_nhwc_small_planes_mixed_classes(oracle, C, HW, dtype):
    """NHWC planes held in registers: channel counts that are multiples of 32 (a wave holds
    channels c, c+8, c+16, c+24: whole-line workgroups) and multiples of 8 only, with angle
    layouts under which the four channels of a wave differ in class or are not canonical at all
    (one pass per class, the table-driven pass among them), odd batch sizes."""
    rng = np.random.default_rng(C + HW)
    _case(oracle, 5, C, HW, HW, 31, 1, dtype, True, grouped_theta(C), seed=C * HW)
    theta = canonical_theta(C)
    theta[1::3] = rng.uniform(-math.pi, 2 * math.pi, len(theta[1::3])).astype(np.float32)
    _case(oracle, 3, C, HW, HW, 31, 1, dtype, True, theta, seed=C * HW + 1)
    theta = canonical_theta(C)[rng.permutation(C)]
    _case(oracle, 2, C, HW, HW, 15, 1, dtype, True, theta, seed=C * HW + 2)


@pytest.mark.parametrize("nhwc", [False, True], ids=["nchw", "nhwc"])
@pytest.mark.parametrize("K", [7, 13, 15, 27, 31])
def test_kernel_sizes_grouped_theta(oracle, K, nhwc):
    """Cropped backbone kernel sizes; contiguous-group angles with the +90deg layer offset."""
    _case(oracle, 2, 72, 20, 24, K, 1, torch.float32, nhwc, grouped_theta(72, 0.5), seed=K)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("nhwc", [False, True], ids=["nchw", "nhwc"])
@pytest.mark.parametrize("stride,H,W,K", [(2, 32, 32, 31), (2, 24, 40, 15), (2, 15, 21, 15),
                                          (4, 32, 24, 7), (2, 7, 9, 31)])
def test_strided_and_odd_extents(oracle, stride, H, W, K, nhwc, dtype):
    """Stem-like strided cases, including extents not divisible by the stride
    (P = ceil(H/stride): the arbitrary-size semantics of dwoconv1d.py:154-187)."""
    _case(oracle, 2, 64, H, W, K, stride, dtype, nhwc, grouped_theta(64), seed=H * W + K)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("stride,H,W,K", [(2, 150, 138, 31), (1, 70, 200, 15), (4, 97, 64, 27)])
def test_nhwc_large_planes_many_tiles(oracle, stride, H, W, K, dtype):
    """NHWC planes that take several bands and sub-tiles per workgroup; the eight canonical
    orientations in channel groups of four plus one group of arbitrary angles (mixed tap extents
    inside a slice)."""
    theta = np.concatenate([np.repeat(canonical_theta(8), 4),
                            np.array([0.3, 1.1, 2.0, 2.9], dtype=np.float32)]).astype(np.float32)
    _case(oracle, 2, 36, H, W, K, stride, dtype, True, theta, seed=H + W + K)


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("stride,H,W,K", [(2, 150, 138, 31), (1, 70, 200, 15), (4, 97, 64, 27),
                                          (2, 61, 35, 31)])
def test_nchw_large_planes_many_tiles(oracle, stride, H, W, K, dtype):
    """NCHW planes without compile-time kernels, several bands and sub-tiles per workgroup, a
    channel count that leaves a partial last group of four; strided dgrad by residue classes."""
    theta = np.concatenate([np.repeat(canonical_theta(8), 4),
                            np.array([0.3, 1.1, 2.0, 2.9, 4.4, -0.7], dtype=np.float32)]).astype(np.float32)
    _case(oracle, 3, 38, H, W, K, stride, dtype, False, theta, seed=H + W + K + 1)


@pytest.mark.parametrize("nhwc", [False, True], ids=["nchw", "nhwc"])
def test_random_angles_ragged_shapes(oracle, nhwc):
    rng = np.random.default_rng(77)
    for (N, C, H, W, K) in [(1, 1, 1, 1, 31), (3, 5, 1, 9, 7), (2, 67, 9, 1, 15), (1, 130, 33, 17, 31),
                            (2, 9, 61, 70, 31), (1, 3, 130, 140, 31)]:
        theta = rng.uniform(-math.pi, 2 * math.pi, C).astype(np.float32)
        _case(oracle, N, C, H, W, K, 1, torch.float32, nhwc, theta, seed=N * C + H)


@pytest.mark.parametrize("nhwc", [False, True], ids=["nchw", "nhwc"])
@pytest.mark.parametrize("stride", [2, 4])
def test_strided_ragged_shapes_random_angles(oracle, stride, nhwc):
    """Strided fprop, dgrad by residue classes and wgrad at degenerate extents (single rows and
    columns, extents below the stride), odd channel counts, random angles."""
    rng = np.random.default_rng(100 + stride)
    for (N, C, H, W, K) in [(1, 1, 1, 1, 31), (2, 3, 1, 9, 7), (2, 6, 9, 1, 15), (1, 9, 3, 2, 31),
                            (2, 12, 33, 17, 31), (1, 4, 70, 61, 27), (3, 8, 5, 130, 13)]:
        if nhwc and C % 4 != 0 and K not in (7, 13, 15, 27, 31):
            continue
        theta = rng.uniform(-math.pi, 2 * math.pi, C).astype(np.float32)
        _case(oracle, N, C, H, W, K, stride, torch.float32, nhwc, theta, seed=N * C + H + stride)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("nhwc", [False, True], ids=["nchw", "nhwc"])
def test_largest_kernel_size(oracle, nhwc, dtype):
    """K = 63, the largest the tap table holds: 16-bit activations run on the tile kernels, fp32
    (whose smallest window would not fit an LDS plane) on the generic ones."""
    rng = np.random.default_rng(63)
    theta = rng.uniform(0, math.pi, 8).astype(np.float32)
    theta[:3] = [0.0, math.pi / 2, math.pi / 4]
    _case(oracle, 2, 8, 40, 37, 63, 1, dtype, nhwc, theta, seed=63)
    _case(oracle, 1, 8, 40, 37, 63, 2, dtype, nhwc, theta, seed=64)


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_randomized_shapes_all_paths(oracle, seed):
    """Seeded random draws over batch, channels, extents, kernel size, stride, element type,
    layout and angle assignment (arbitrary, round-robin canonical, grouped canonical): every
    routing decision of the C ABI gets exercised at shapes nobody picked by hand."""
    rng = np.random.default_rng(seed)
    for it in range(40):
        nhwc = bool(rng.integers(2))
        K = int(rng.choice([3, 7, 13, 15, 27, 31, 45, 63]))
        stride = int(rng.choice([1, 1, 2, 4]))
        N = int(rng.integers(1, 4))
        C = int(rng.choice([1, 2, 3, 4, 5, 8, 12, 17, 32, 36]))
        H, W = int(rng.integers(1, 90)), int(rng.integers(1, 150))
        if rng.integers(4) == 0:
            H, W = W, H
        dtype = DTYPES[int(rng.integers(3))]
        kind = int(rng.integers(3))
        if kind == 0:
            theta = rng.uniform(-math.pi, 2 * math.pi, C).astype(np.float32)
        elif kind == 1:
            theta = canonical_theta(C)
        else:
            theta = grouped_theta(C)
        _case(oracle, N, C, H, W, K, stride, dtype, nhwc, theta, seed=seed * 1000 + it)


@pytest.mark.parametrize("nhwc", [False, True], ids=["nchw", "nhwc"])
@pytest.mark.parametrize("C,HW", [(96, 56), (192, 28), (384, 14), (768, 7)])
def test_wgrad_is_deterministic_on_both_reduction_paths(C, HW, nhwc):
    """The partial sums of a channel are added in a fixed order, by the last workgroup of the
    channel to finish (found through an integer counter) or by a second kernel: repeated calls
    and the two paths must agree bit for bit, at the four stage shapes in both layouts."""
    from oriented1d_amd import _lib

    lib = _lib.ready(torch.device("cuda:0"))
    K, N = 31, 32
    g = torch.Generator(device="cuda").manual_seed(5 + HW)
    shape = (N, HW, HW, C) if nhwc else (N, C, HW, HW)
    x = torch.randn(shape, device="cuda", generator=g)
    dy = torch.randn(shape, device="cuda", generator=g)
    taps = op.build_taps(torch.from_numpy(canonical_theta(C)), C, K).cuda()
    print("determinism C%d %dx%d %s" % (C, HW, HW, "nhwc" if nhwc else "nchw"), flush=True)
    a, adb = op.wgrad(dy, x, taps, K, nhwc=nhwc, with_bias=True)
    for rep in range(4):
        b, bdb = op.wgrad(dy, x, taps, K, nhwc=nhwc, with_bias=True)
        assert torch.equal(a, b) and torch.equal(adb, bdb), rep
    prev = lib.dwo_set_wgrad_reduction(0)  # second-kernel reduction
    try:
        assert prev == 1
        c, cdb = op.wgrad(dy, x, taps, K, nhwc=nhwc, with_bias=True)
        torch.cuda.synchronize()
    finally:
        lib.dwo_set_wgrad_reduction(1)
    assert torch.equal(a, c) and torch.equal(adb, cdb)
    d, ddb = op.wgrad(dy, x, taps, K, nhwc=nhwc, with_bias=True)  # the counters are back at zero
    assert torch.equal(a, d) and torch.equal(adb, ddb)


def test_wgrad_with_more_channels_than_a_counter_row(oracle):
    """NCHW with more channels than a row of the library's counters holds (4096): the plane
    kernel writes plain partial sums and the second kernel adds them."""
    _case(oracle, 8, 4104, 7, 7, 31, 1, torch.float32, False, canonical_theta(4104), seed=4104)


def test_wgrad_on_two_streams_at_once():
    """Overlapping wgrad calls on two streams with their own scratch and outputs: each stream
    counts on its own counters, so both give the single-stream result, call after call."""
    from oriented1d_amd import _lib

    _lib.ready(torch.device("cuda:0"))
    C, K, HW, N = 192, 31, 28, 64
    g = torch.Generator(device="cuda").manual_seed(9)
    taps = op.build_taps(torch.from_numpy(canonical_theta(C)), C, K).cuda()
    data = [(torch.randn(N, C, HW, HW, device="cuda", generator=g),
             torch.randn(N, C, HW, HW, device="cuda", generator=g)) for _ in range(2)]
    ref = [op.wgrad(dy, x, taps, K, with_bias=True) for x, dy in data]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    got = [[], []]
    for rep in range(12):
        for k, st in enumerate(streams):
            with torch.cuda.stream(st):
                x, dy = data[k]
                got[k].append(op.wgrad(dy, x, taps, K, with_bias=True))
    torch.cuda.synchronize()
    for k in range(2):
        for dw, db in got[k]:
            assert torch.equal(dw, ref[k][0]) and torch.equal(db, ref[k][1])


@pytest.mark.parametrize("nhwc", [False, True], ids=["nchw", "nhwc"])
def test_batch_128_bf16(oracle, nhwc):
    """Batch 128, the batch the inference configuration runs at: all three operators of the
    first stage's shape against the oracle."""
    _case(oracle, 128, 96, 56, 56, 31, 1, torch.bfloat16, nhwc, grouped_theta(96), seed=128,
          threads=min(16, oracle.max_threads()))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("nhwc", [False, True], ids=["nchw", "nhwc"])
@pytest.mark.parametrize("C,HW", [(96, 56), (192, 28), (384, 14), (768, 7)])
def test_full_size_all_ops_against_oracle(oracle, C, HW, nhwc, dtype):
    """Batch-64 stage shapes, the tensors the roofline is measured on: every image of fprop and
    dgrad (all image groups of every workgroup split, first and last batch included) and the
    full-length wgrad / bias-gradient reduction against the double-accumulating oracle, plus
    the size-independent properties (adjoint identities, exact linearity)."""
    N, K = 64, 31
    theta = canonical_theta(C)
    rng = np.random.default_rng(C + HW)
    x = rounded(rng.standard_normal((N, C, HW, HW)).astype(np.float32), dtype)
    dy = rounded(rng.standard_normal((N, C, HW, HW)).astype(np.float32), dtype)
    w = (rng.standard_normal((C, 1, 1, K)) * 0.02).astype(np.float32)
    print("full size C%d %dx%d %s %s" % (C, HW, HW, dtype, "nhwc" if nhwc else "nchw"), flush=True)

    def lay(a):
        return np.ascontiguousarray(a.transpose(0, 2, 3, 1)) if nhwc else a

    def unlay(t):
        return t.permute(0, 3, 1, 2) if nhwc else t

    taps = op.build_taps(torch.from_numpy(theta), C, K).cuda()
    xd, dyd, wd = dev(lay(x), dtype), dev(lay(dy), dtype), dev(w, torch.float32)
    yd = op.fprop(xd, wd, taps, nhwc=nhwc)
    dxd = op.dgrad(dyd, wd, taps, (HW, HW), nhwc=nhwc)
    dwd, dbd = op.wgrad(dyd, xd, taps, K, nhwc=nhwc, with_bias=True)
    torch.cuda.synchronize()
    nthr = min(16, oracle.max_threads())
    assert_close(host(unlay(yd)), oracle.fprop(x, w, theta, threads=nthr), dtype, "fprop")
    assert_close(host(unlay(dxd)), oracle.dgrad(dy, w, theta, threads=nthr), dtype, "dgrad")
    # dw/db are fp32 sums of exact products of the (already rounded) inputs: fp32 tolerance
    assert_close(host(dwd), oracle.wgrad(dy, x, theta, K, threads=nthr), torch.float32, "wgrad")
    assert_close(host(dbd), oracle.bgrad(dy), torch.float32, "bgrad")
    # <y,dy> = <x,dx> = <w,dw>; terms are O(1) random so compare against sqrt(#terms) scale
    a = (yd.double() * dyd.double()).sum().item()
    b = (xd.double() * dxd.double()).sum().item()
    c = (wd.double() * dwd.double()).sum().item()
    scale = math.sqrt((yd.double() ** 2).sum().item() * (dyd.double() ** 2).sum().item())
    tol = TOL[dtype]
    assert abs(a - c) <= tol * scale and abs(a - b) <= tol * scale, (a, b, c, scale)
    # linearity: fprop(2x) = 2 fprop(x) exactly (power-of-two scaling commutes with rounding)
    assert torch.equal(op.fprop(xd * 2, wd, taps, nhwc=nhwc), yd * 2)


# The operator launches of the two training configurations, at reduced batch, bf16 (what the
# networks run under autocast / after .to(bfloat16)): ConvNeXt-B-1D++ at 224 x 224 -- second
# convolutions NHWC K=31 with a residual tap on the 4x-expanded channels, first convolutions
# NCHW K=15, the K=15 stem -- and ConvNeXt-T-1D at 512 x 512 -- stages of 128, 64, 32, 16
# squared and the K=31 stem.  Angles are the networks' contiguous groups, odd layers turned by
# 90 degrees (models/convnext.py:60-77).
_TRAINING_LAUNCHES = [
    # N, C, HW, K, stride, nhwc
    (2, 512, 56, 31, 1, True), (2, 1024, 28, 31, 1, True), (2, 2048, 14, 31, 1, True),
    (3, 4096, 7, 31, 1, True),
    (2, 128, 56, 15, 1, False), (2, 256, 28, 15, 1, False), (2, 512, 14, 15, 1, False),
    (3, 1024, 7, 15, 1, False),
    (2, 64, 224, 15, 2, True), (2, 64, 112, 15, 2, True),
    (2, 96, 128, 31, 1, False), (2, 192, 64, 31, 1, False), (2, 384, 32, 31, 1, False),
    (3, 768, 16, 31, 1, False),
    (1, 64, 512, 31, 2, True), (2, 64, 256, 31, 2, True), (2, 64, 224, 31, 2, True),
    (2, 64, 112, 31, 2, True),  # second stem convolution of ConvNeXt-T-1D at 224 x 224
]


@pytest.mark.parametrize("offset", [0.0, 0.5], ids=["even", "odd"])
@pytest.mark.parametrize("N,C,HW,K,stride,nhwc", _TRAINING_LAUNCHES,
                         ids=["%dx%d_k%d_s%d_%s" % (c, hw, k, s, "nhwc" if l else "nchw")
                              for _, c, hw, k, s, l in _TRAINING_LAUNCHES])
def test_training_configuration_launch_shapes(oracle, N, C, HW, K, stride, nhwc, offset):
    if offset == 0.5 and HW > 128:
        pytest.skip("the two stem layers differ by the same 90 degrees; one is enough at this size")
    _case(oracle, N, C, HW, HW, K, stride, torch.bfloat16, nhwc, grouped_theta(C, offset),
          seed=C + HW + K, threads=min(16, oracle.max_threads()))


@pytest.mark.gpu
def test_step_captured_in_a_graph_replays_identically():
    """fprop + dgrad + wgrad through the C ABI captured into one graph.  The first thing the
    capture contains is the first call of each entry point in this process for this shape: the
    per-device set-up (occupancy queries, kernel attributes) was done by dwo_init, so the calls
    only launch kernels.  Three replays, each after unrelated eager work and
    a synchronisation, on fresh inputs written into the captured buffers, must equal the eager
    results bit for bit."""
    torch.manual_seed(5)
    N, C, HW, K = 4, 80, 28, 15  # a (K, extent) no other test of this module launches first
    theta = torch.from_numpy(canonical_theta(C))
    taps = op.build_taps(theta, C, K).cuda()
    w = (torch.randn(C, 1, 1, K, device="cuda") * 0.02)
    x = torch.randn(N, C, HW, HW, device="cuda")
    dy = torch.randn(N, C, HW, HW, device="cuda")
    stream = torch.cuda.Stream()
    from oriented1d_amd import _lib
    _lib.ready(x.device)
    with torch.cuda.stream(stream):
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            gy = op.fprop(x, w, taps, 1)
            gdx = op.dgrad(dy, w, taps, (HW, HW), 1)
            gdw, gdb = op.wgrad(dy, x, taps, K, 1, with_bias=True)
        for rep in range(3):
            x.copy_(torch.randn_like(x))
            dy.copy_(torch.randn_like(dy))
            junk = (torch.randn(1 << 20, device="cuda") * 2).sum()  # eager work in between
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            ey = op.fprop(x, w, taps, 1)
            edx = op.dgrad(dy, w, taps, (HW, HW), 1)
            edw, edb = op.wgrad(dy, x, taps, K, 1, with_bias=True)
            torch.cuda.synchronize()
            assert torch.equal(gy, ey) and torch.equal(gdx, edx), rep
            assert torch.equal(gdw, edw) and torch.equal(gdb, edb), rep
            assert torch.isfinite(junk)
