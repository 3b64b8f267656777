"""The forward-only glue kernels against the PyTorch passes they replace
(models/convnext.py:306-318 and :176-190): LayerNorm over channels with and without the layout
change, exact GELU, layer scale + transpose + residual.  Tolerances: fp32 1e-5, 16-bit 1e-2
(tensor-level, as for the operator)."""
import pytest
import torch
import torch.nn.functional as F

from parity_util import TOL, rel_err

from oriented1d_amd import fused

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16, torch.float16]


def _close(got, ref, dtype, what):
    e_max, e_l2 = rel_err(got.float().cpu().numpy(), ref.double().cpu().numpy())
    assert e_max <= TOL[dtype] and e_l2 <= TOL[dtype], (what, e_max, e_l2)


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("N,C,H,W", [(2, 96, 56, 56), (3, 192, 28, 28), (2, 384, 14, 14),
                                     (2, 768, 7, 7), (1, 1024, 7, 7), (2, 64, 9, 13), (1, 6, 3, 5)])
def test_nchw_layernorm_nhwc(N, C, H, W, dtype):
    torch.manual_seed(C + H)
    x = (torch.randn(N, C, H, W, device="cuda") * 2 + 0.5).to(dtype)
    g = torch.randn(C, device="cuda") * 0.5 + 1
    b = torch.randn(C, device="cuda") * 0.1
    got = fused.nchw_layernorm_nhwc(x, g, b, 1e-6)
    ref = F.layer_norm(x.double().permute(0, 2, 3, 1), (C,), g.double(), b.double(), 1e-6)
    assert got.shape == (N, H, W, C) and got.dtype == dtype and got.is_contiguous()
    _close(got, ref, dtype, "nchw_layernorm_nhwc")


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("gelu", [False, True])
@pytest.mark.parametrize("shape", [(2, 112, 112, 64), (3, 14, 14, 384), (5, 7, 7, 1536), (7, 2048),
                                   (1, 3, 5, 2)])
def test_layernorm_nhwc(shape, gelu, dtype):
    torch.manual_seed(shape[-1])
    C = shape[-1]
    x = (torch.randn(*shape, device="cuda") * 3 - 0.25).to(dtype)
    g = torch.randn(C, device="cuda") * 0.5 + 1
    b = torch.randn(C, device="cuda") * 0.1
    got = fused.layernorm_nhwc(x, g, b, 1e-6, gelu=gelu)
    ref = F.layer_norm(x.double(), (C,), g.double(), b.double(), 1e-6)
    if gelu:
        ref = F.gelu(ref)
    assert got.shape == x.shape and got.dtype == dtype
    _close(got, ref, dtype, "layernorm_nhwc")


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("with_scale,with_res", [(True, True), (False, False), (True, False)])
@pytest.mark.parametrize("N,C,H,W", [(2, 96, 56, 56), (2, 768, 7, 7), (3, 64, 9, 13), (1, 1536, 2, 3)])
def test_nhwc_scale_add_nchw(N, C, H, W, with_scale, with_res, dtype):
    torch.manual_seed(C + W)
    y = torch.randn(N, H, W, C, device="cuda").to(dtype)
    s = torch.randn(C, device="cuda") if with_scale else None
    r = torch.randn(N, C, H, W, device="cuda").to(dtype) if with_res else None
    got = fused.nhwc_scale_add_nchw(y, s, r)
    ref = y.double()
    if with_scale:
        ref = ref * s.double()
    ref = ref.permute(0, 3, 1, 2)
    if with_res:
        ref = ref + r.double()
    assert got.shape == (N, C, H, W) and got.is_contiguous()
    _close(got, ref, dtype, "nhwc_scale_add_nchw")


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("Cin,C,H,W,K,stride", [(3, 64, 64, 48, 31, 2), (3, 24, 37, 29, 15, 2),
                                               (4, 8, 20, 20, 7, 1), (1, 16, 33, 70, 31, 4),
                                               (3, 64, 224, 224, 31, 2)])  # the stem's own shape
def test_pointwise_then_oriented_conv(oracle, Cin, C, H, W, K, stride, dtype):
    """dwo_pointwise_fprop_nhwc against the two separate layers: nn.Linear Cin -> C rounded to
    the activation type (what the reference's pw1 hands to dw1, models/convnext.py:177-178),
    then the oracle's fprop with bias."""
    import numpy as np
    from parity_util import grouped_theta, rounded
    from oriented1d_amd.dwoconv1d import DepthwiseOrientedConv1d

    torch.manual_seed(Cin * 100 + C)
    lin = torch.nn.Linear(Cin, C).cuda()
    conv = DepthwiseOrientedConv1d(C, C, K, groups=C, stride=stride, padding=K // 2, bias=True,
                                   angle=grouped_theta(C).tolist(), nhwc=True).cuda()
    torch.nn.init.normal_(conv.bias, std=0.3)
    x = torch.randn(2, H, W, Cin, device="cuda").to(dtype)
    with torch.no_grad():
        got = fused.pointwise_dwconv_nhwc(x, lin, conv)
    mid = x.double().cpu().numpy() @ lin.weight.detach().double().cpu().numpy().T \
        + lin.bias.detach().double().cpu().numpy()
    mid = rounded(mid.astype(np.float32), dtype)  # the separate layer's output in the tensor's type
    ref = oracle.fprop(np.ascontiguousarray(mid.transpose(0, 3, 1, 2)),
                       conv.weight.detach().cpu().numpy(), conv.theta.detach().cpu().numpy(), stride)
    ref = ref + conv.bias.detach().double().cpu().numpy().reshape(1, -1, 1, 1)
    P, Q = -(-H // stride), -(-W // stride)
    assert got.shape == (2, P, Q, C) and got.dtype == dtype
    _close(got.permute(0, 3, 1, 2), torch.from_numpy(ref), dtype, "pointwise_fprop")


def test_argument_errors():
    x = torch.randn(2, 7, 4, 4, device="cuda")  # odd channel count
    with pytest.raises(RuntimeError):
        fused.nchw_layernorm_nhwc(x, torch.ones(7), torch.zeros(7), 1e-6)
    assert not fused.usable(x, 7, tiled=True)
    assert not fused.usable(torch.randn(2, 8, 4, 4), 8, tiled=True)  # CPU tensor
    w = torch.randn(2, 8, 4, 4, device="cuda", requires_grad=True)
    assert not fused.usable(w, 8, tiled=True)
    with torch.no_grad():
        assert fused.usable(w, 8, tiled=True)


@pytest.mark.parametrize("variant", ["1d", "1dpp"])
def test_block_and_stem_fused_equal_unfused(variant):
    """Block-level parity: the harness in no-grad eval mode (fused glue) against the same
    modules with autograd on (PyTorch composition)."""
    from oriented1d_amd.convnext1d import ConvNeXt1D

    torch.manual_seed(3)
    m = ConvNeXt1D(depths=(1, 1, 1, 1), dims=(16, 32, 64, 128), variant=variant, stem_dim1=24,
                   num_classes=10, layer_scale_init_value=1.0).cuda().eval()
    for name, p in m.named_parameters():
        if name.endswith("bias") or "norm" in name:
            torch.nn.init.normal_(p, mean=0.3, std=0.2)
    x = torch.randn(2, 3, 64, 64, device="cuda")
    with torch.no_grad():
        y_fused = m(x)
    y_plain = m(x.requires_grad_(True))  # gradient recording switches the glue kernels off
    _close(y_fused, y_plain.detach(), torch.float32, "network")


def test_bf16_network_fused_equal_unfused_and_parameter_copies_refresh():
    """The 16-bit network (parameters cast with .bfloat16(): the library works from cached fp32
    copies of them) with and without the glue kernels, and the copies follow in-place updates."""
    from oriented1d_amd.convnext1d import ConvNeXt1D

    torch.manual_seed(4)
    m = ConvNeXt1D(depths=(1, 1, 1, 1), dims=(16, 32, 64, 128), variant="1d", stem_dim1=24,
                   num_classes=10, layer_scale_init_value=1.0).cuda().bfloat16().eval()
    x = torch.randn(2, 3, 64, 64, device="cuda").bfloat16()
    with torch.no_grad():
        y_fused = m(x)
    y_plain = m(x.requires_grad_(True)).detach()
    _close(y_fused, y_plain, torch.bfloat16, "bf16 network")
    with torch.no_grad():
        m.stages[0][0].dwconv.weight.mul_(3.0)   # in-place update: the cached copy must refresh
        y_fused2 = m(x.detach())
    y_plain2 = m(x).detach()
    _close(y_fused2, y_plain2, torch.bfloat16, "bf16 network after update")
    assert not torch.equal(y_fused, y_fused2)
