"""ConvNeXt-1D / 1D++ harness: structural known answers on CPU (parameter counts published in
the reference's README.md:41-46, state_dict naming of models/convnext.py) and, on the GPU, the
whole network against the same network with every oriented conv computed by the CPU oracle."""
import numpy as np
import pytest
import torch

from oriented1d_amd.convnext1d import (ConvNeXt1D, channel_angles, convnext_base_1d,
                                       convnext_tiny_1d)
from oriented1d_amd.dwoconv1d import DepthwiseOrientedConv1d


@pytest.mark.parametrize("factory,variant,millions", [
    (convnext_tiny_1d, "1d", 28.5), (convnext_tiny_1d, "1dpp", 29.2),
    (convnext_base_1d, "1d", 88.0), (convnext_base_1d, "1dpp", 90.0)])
def test_parameter_counts_match_published(factory, variant, millions):
    n = sum(p.numel() for p in factory(variant=variant).parameters())
    assert abs(n / 1e6 - millions) < 0.45, n


def test_state_dict_layout_and_angles():
    m = convnext_tiny_1d(variant="1dpp")
    sd = m.state_dict()
    for key in ("downsample_layers.0.pw1.weight", "downsample_layers.0.dw1.theta",
                "downsample_layers.0.norm3.bias", "downsample_layers.1.0.weight",
                "downsample_layers.1.1.weight", "stages.0.0.dwconv1.weight",
                "stages.0.0.dwconv2.theta", "stages.2.8.pwconv2.bias", "stages.3.2.gamma",
                "norm.weight", "head.bias"):
        assert key in sd, key
    assert tuple(sd["stages.0.0.dwconv1.weight"].shape) == (96, 1, 1, 15)
    assert tuple(sd["stages.0.0.dwconv2.weight"].shape) == (384, 1, 1, 31)
    assert tuple(sd["downsample_layers.0.dw1.weight"].shape) == (64, 1, 1, 15)
    m1 = convnext_tiny_1d(variant="1d")
    assert "stages.1.1.dwconv.bias" in m1.state_dict()
    assert tuple(m1.state_dict()["downsample_layers.0.dw2.weight"].shape) == (64, 1, 1, 31)
    # contiguous groups of C/8 channels per direction; +90 degrees on odd layers
    a = channel_angles(96)
    assert a[0] == 0.0 and a[11] == 0.0 and abs(a[12] - np.pi / 8) < 1e-12 and abs(a[95] - 7 * np.pi / 8) < 1e-12
    th0, th1 = m1.stages[0][0].dwconv.theta, m1.stages[0][1].dwconv.theta
    assert torch.allclose((th0 + np.pi / 2) % np.pi, th1 % np.pi, atol=1e-6)
    assert m1.stages[0][0].dwconv.nhwc is False and m.stages[0][0].dwconv2.nhwc is True
    assert m.stages[0][0].dwconv2.resid is not None and m.downsample_layers[0].dw1.stride == (2, 2)


@pytest.mark.parametrize("variant", ["1d", "1dpp"])
def test_backbone_form_and_checkpoint_conversion(variant):
    """Backbone form: wrapped operator names, per-stage cropped kernels
    (semantic_segmentation/backbone/convnext.py:74-80,316-327), and the converter: every tensor of
    the classification checkpoint arrives under its wrapped name, kernels are cropped around the
    centre tap (the cropped operator equals the original restricted to its inner taps)."""
    from oriented1d_amd.backbone_weights import centre_crop_kernel, convert_to_backbone_state_dict

    torch.manual_seed(1)
    cls = ConvNeXt1D(depths=(1, 1, 1, 1), dims=(8, 16, 24, 32), variant=variant, stem_dim1=8,
                     num_classes=5)
    bb = ConvNeXt1D(depths=(1, 1, 1, 1), dims=(8, 16, 24, 32), variant=variant, stem_dim1=8,
                    backbone=True)
    want = {"1d": [(31,), (31,), (27,), (13,)], "1dpp": [(15, 31), (15, 31), (15, 27), (13, 13)]}[variant]
    for i in range(4):
        blk = bb.stages[i][0]
        convs = [blk.dwconv1, blk.dwconv2] if variant == "1dpp" else [blk.dwconv]
        assert tuple(c.conv.kernel_size[1] for c in convs) == want[i]
        assert all(c.conv.arbitrary_size for c in convs)
    conv = convert_to_backbone_state_dict(cls.state_dict(), bb.state_dict())
    missing, unexpected = bb.load_state_dict(conv, strict=False)
    assert not unexpected
    assert all(k.startswith("norm") for k in missing), missing  # the four per-stage output norms
    src = cls.state_dict()
    last = "stages.3.0.dwconv2" if variant == "1dpp" else "stages.3.0.dwconv"
    w_src, w_dst = src[last + ".weight"], bb.state_dict()[last + ".conv.weight"]
    K, k = w_src.shape[-1], w_dst.shape[-1]
    assert k == 13 and torch.equal(w_dst, w_src[..., (K - k) // 2:(K + k) // 2])
    assert torch.equal(bb.state_dict()[last + ".conv.theta"], src[last + ".theta"])
    assert torch.equal(bb.state_dict()["stages.0.0.pwconv1.weight"], src["stages.0.0.pwconv1.weight"])
    w = torch.arange(2 * 7, dtype=torch.float32).reshape(2, 1, 1, 7)
    assert centre_crop_kernel(w, 3)[0, 0, 0].tolist() == [2.0, 3.0, 4.0]
    with pytest.raises(ValueError):
        centre_crop_kernel(w, 4)


@pytest.mark.gpu
def test_backbone_runs_on_odd_input_sizes():
    torch.manual_seed(0)
    m = ConvNeXt1D(depths=(1, 1, 1, 1), dims=(8, 16, 24, 32), variant="1d", stem_dim1=8,
                   backbone=True).cuda().eval()
    with torch.no_grad():
        outs = m(torch.randn(1, 3, 72, 104, device="cuda"))
    assert [tuple(o.shape) for o in outs] == [(1, 8, 18, 26), (1, 16, 9, 13), (1, 24, 4, 6), (1, 32, 2, 3)]
    assert all(torch.isfinite(o).all() for o in outs)


@pytest.mark.gpu
@pytest.mark.parametrize("variant", ["1d", "1dpp"])
def test_network_matches_oracle_composition(oracle, variant):
    torch.manual_seed(0)
    m = ConvNeXt1D(depths=(1, 2, 1, 1), dims=(16, 32, 64, 128), variant=variant, stem_dim1=24,
                   num_classes=10, layer_scale_init_value=1.0).cuda().eval()
    for name, p in m.named_parameters():  # biases away from their zero defaults
        if name.endswith("bias"):
            torch.nn.init.normal_(p, std=0.1)
    x = torch.randn(2, 3, 64, 64, device="cuda")
    with torch.no_grad():
        y = m(x)

    def oracle_forward(mod):
        def fwd(t):
            w = mod.weight.detach().float().cpu().numpy()
            b = mod.bias.detach().float().cpu().numpy()
            th = mod.theta.detach().float().cpu().numpy()
            out = oracle.module_forward(t.detach().float().cpu().numpy(), w, th, bias=b,
                                        stride=mod.stride[0], nhwc=mod.nhwc,
                                        resid=mod.resid is not None)
            return torch.from_numpy(out).to(device=t.device, dtype=t.dtype)
        return fwd

    for mod in m.modules():
        if isinstance(mod, DepthwiseOrientedConv1d):
            mod.forward = oracle_forward(mod)
    with torch.no_grad():
        y_ref = m(x)
    err = (y - y_ref).abs().max().item() / y_ref.abs().max().item()
    assert y.shape == (2, 10) and err < 2e-5, err


@pytest.mark.gpu
@pytest.mark.parametrize("variant", ["1d", "1dpp"])
def test_bf16_network_against_fp32_oracle_composition(oracle, variant):
    """The 16-bit inference network (what the images-per-second figure runs) against an
    independent result: the same weights in fp32 with every oriented convolution evaluated by
    the oracle.  bf16 rounding accumulates over the layers, so the gate is 3e-2 of the output
    scale (a wrong tap, weight or layout anywhere is an error of order one)."""
    torch.manual_seed(7)
    m = ConvNeXt1D(depths=(1, 2, 1, 1), dims=(16, 32, 64, 128), variant=variant, stem_dim1=24,
                   num_classes=10, layer_scale_init_value=1.0).cuda().eval()
    for name, p in m.named_parameters():
        if name.endswith("bias"):
            torch.nn.init.normal_(p, std=0.1)
    x = torch.randn(2, 3, 64, 64, device="cuda")
    import copy
    m16 = copy.deepcopy(m).bfloat16()
    with torch.no_grad():
        y16 = m16(x.bfloat16()).float()

    def oracle_forward(mod):
        def fwd(t):
            out = oracle.module_forward(t.detach().float().cpu().numpy(),
                                        mod.weight.detach().float().cpu().numpy(),
                                        mod.theta.detach().float().cpu().numpy(),
                                        bias=mod.bias.detach().float().cpu().numpy(),
                                        stride=mod.stride[0], nhwc=mod.nhwc,
                                        resid=mod.resid is not None)
            return torch.from_numpy(out).to(device=t.device, dtype=t.dtype)
        return fwd

    for mod in m.modules():
        if isinstance(mod, DepthwiseOrientedConv1d):
            mod.forward = oracle_forward(mod)
    with torch.no_grad():
        y_ref = m(x)
    err = (y16 - y_ref).abs().max().item() / y_ref.abs().max().item()
    assert y16.shape == (2, 10) and torch.isfinite(y16).all() and err < 3e-2, err


@pytest.mark.gpu
def test_training_step_and_stage_outputs():
    torch.manual_seed(1)
    m = ConvNeXt1D(depths=(1, 1, 1, 1), dims=(16, 32, 64, 128), variant="1dpp", stem_dim1=16,
                   out_stages=True, drop_path_rate=0.2).cuda().train()
    x = torch.randn(2, 3, 64, 64, device="cuda")
    with torch.autocast("cuda", dtype=torch.bfloat16):
        outs = m(x)
    assert [tuple(o.shape[1:]) for o in outs] == [(16, 16, 16), (32, 8, 8), (64, 4, 4), (128, 2, 2)]
    sum(o.float().square().mean() for o in outs).backward()
    for name, p in m.named_parameters():
        if name.endswith("theta"):
            assert p.grad is None, name
        else:
            assert p.grad is not None and torch.isfinite(p.grad).all(), name


@pytest.mark.gpu
@pytest.mark.parametrize("variant,autocast", [("1dpp", True), ("1dpp", False), ("1d", True)])
def test_training_step_gradients_match_oracle(oracle, variant, autocast):
    """One forward + backward + AdamW step of a reduced network, as the training configurations
    run it (bf16 autocast over fp32 master weights, or plain fp32).  Every oriented convolution's
    input, upstream gradient and the three gradients it produced are captured; each is checked
    against the oracle's module_backward on the captured tensors (dwoconv1d.py:41-69)."""
    from parity_util import assert_close, host

    torch.manual_seed(3)
    net = ConvNeXt1D(depths=(1, 2, 1, 1), dims=(16, 32, 64, 128), variant=variant, stem_dim1=16,
                     num_classes=10, layer_scale_init_value=1.0).cuda().train()
    for name, p in net.named_parameters():
        if name.endswith("bias"):
            torch.nn.init.normal_(p, std=0.1)
    opt = torch.optim.AdamW(net.parameters(), lr=1e-3, weight_decay=0.05)
    convs = [(n, m) for n, m in net.named_modules() if isinstance(m, DepthwiseOrientedConv1d)]
    seen = {}

    def capture_input(name):
        # the convolution gets its own copy of the input, so the gradient seen on that copy is
        # the convolution's dx alone (the block's residual branch reads the original)
        def pre_hook(mod, inputs):
            xi = inputs[0].clone()
            rec = seen.setdefault(name, {})
            rec["x"] = xi.detach().clone()
            if xi.requires_grad:
                xi.register_hook(lambda g: rec.__setitem__("dx", g.detach().clone()))
            return (xi,)
        return pre_hook

    def capture_output(name):
        def hook(mod, inputs, output):
            rec = seen[name]
            output.register_hook(lambda g: rec.__setitem__("dy", g.detach().clone()))
        return hook

    handles = [m.register_forward_pre_hook(capture_input(n)) for n, m in convs]
    handles += [m.register_forward_hook(capture_output(n)) for n, m in convs]
    imgs = torch.randn(4, 3, 64, 64, device="cuda")
    labels = torch.randint(0, 10, (4,), device="cuda")
    before = {n: m.weight.detach().clone() for n, m in convs}
    opt.zero_grad(set_to_none=True)
    with torch.autocast("cuda", dtype=torch.bfloat16, enabled=autocast):
        loss = torch.nn.functional.cross_entropy(net(imgs).float(), labels)
    loss.backward()
    for h in handles:
        h.remove()
    assert len(seen) == len(convs) >= 7
    for name, m in convs:
        rec = seen[name]
        dt = rec["x"].dtype
        w, th = host(before[name]), host(m.theta)
        dx, dw, db = oracle.module_backward(host(rec["dy"]), host(rec["x"]), w, th,
                                            stride=m.stride[0], nhwc=m.nhwc,
                                            resid=m.resid is not None)
        tag = "%s %s %s" % (variant, name, dt)
        assert m.weight.grad.dtype == torch.float32 and m.theta.grad is None
        # dw/db: fp32 sums of products of the captured (already rounded) tensors
        assert_close(host(m.weight.grad), dw, torch.float32, tag + " dw")
        assert_close(host(m.bias.grad), db, torch.float32, tag + " db")
        if "dx" in rec:
            assert_close(host(rec["dx"]), dx, dt, tag + " dx")
    opt.step()
    for name, m in convs:
        assert torch.isfinite(m.weight).all() and not torch.equal(m.weight.detach(), before[name])
