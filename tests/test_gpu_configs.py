"""The benchmark configurations at their own workloads (shape AND dtype), against the CPU oracle where it
finishes in seconds (slices of images, subsets of points, the full-batch filter gradient) and through
size-independent properties for the rest.

  configuration 2, bfloat16 leg   N=64 C=144 56x56, scope 4x4
  configuration 3                 GlobalDeformKernel2d N=128 C=256 28x28, scope 5x5, float16
  configuration 5, sampler leg    nd_linear_sample, data [64, 32, 32, 32], 2^20 points, float32

Tolerances: 16-bit types 1e-2 of the expected tensor's largest magnitude, against the float32 oracle on
the rounded inputs; float32 forward 1e-5, reductions 1e-4 against the float64 oracle.
"""
import numpy as np
import pytest
import torch

from _cases import make_local, mixed_err, rel_err
from oracle import dk_oracle as orc

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _within(err, tol, what=""):
    # the error is computed first, so a failure reports two numbers and not the tensors
    assert err < tol, "%s: error %.3e, tolerance %.0e" % (what, err, tol)


def test_config2_bfloat16_at_full_size():
    from deformable_kernels.ops.deform_kernel.functions import sample_depthwise
    x, wt, rot, gout, cfg = make_local(64, 144, 56, 56, 3, (4, 4), 1, 1, 1, 1, 1.0, seed=0, dtype=torch.bfloat16)
    xg, rg, wg = [t.to(DEV).requires_grad_() for t in (x, rot, wt)]
    args = ((3, 3), (1, 1), (1, 1), (1, 1), 1)
    out = sample_depthwise(xg, rg, wg, *args)
    out.backward(gout.to(DEV))
    torch.cuda.synchronize()
    assert out.dtype == xg.grad.dtype == rg.grad.dtype == wg.grad.dtype == torch.bfloat16
    f = lambda t: t.float().numpy()  # the oracle sees the rounded inputs
    for n in (0, 37, 63):
        sl = slice(n, n + 1)
        want = orc.sample_depthwise_forward(f(x[sl]), f(rot[sl]), f(wt), **cfg)
        gin, grot, _ = orc.sample_depthwise_backward(f(gout[sl]), f(x[sl]), f(rot[sl]), f(wt), **cfg)
        _within(rel_err(out[sl].detach().float().cpu(), want), 1e-2, ("forward", n))
        _within(rel_err(xg.grad[sl].float().cpu(), gin), 1e-2, ("grad input", n))
        _within(rel_err(rg.grad[sl].float().cpu(), grot), 1e-2, ("grad rotation", n))
    # the filter gradient sums over the whole batch: full-batch float32 oracle
    _, _, gw = orc.sample_depthwise_backward(f(gout), f(x), f(rot), f(wt), **cfg)
    _within(rel_err(wg.grad.float().cpu(), gw), 1e-2, "grad filter")


def _global_module(dtype, seed):
    from deformable_kernels.modules import GlobalDeformKernel2d
    torch.manual_seed(seed)
    m = GlobalDeformKernel2d((5, 5), 256, 256, kernel_size=3, stride=1, padding=1, groups=256)
    with torch.no_grad():
        # configuration 3: the pooled branch predicts offsets ~ N(0, 0.5); the inputs' channel means
        # are ~ N(0, 1/28), so a weight of std 14 / sqrt(256) over 256 channels gives them that spread
        m.fc.weight.normal_(0.0, 14.0 / 16.0)
        m.fc.bias.normal_(0.0, 0.1)
    return m.to(DEV).to(dtype)


def test_config3_global_deform_kernel_float16_at_full_size():
    """N=128, C=256, 28x28, scope 5x5, float16, one offset set per image.  The oracle applies the local
    operator with each image's 18 offsets repeated over its pixels (which is what the layer computes:
    the kernels are sampled once per (image, channel), then a depthwise convolution runs), on two
    images for the forward and input gradient and on the full batch for the parameter gradients."""
    N, C, H = 128, 256, 28
    g = torch.Generator().manual_seed(3)
    x = torch.randn(N, C, H, H, generator=g).half()
    gout = torch.randn(N, C, H, H, generator=g).half()
    m = _global_module(torch.float16, seed=30)
    m.fused = True  # first the route that hands each image's offsets to the local operator
    xg = x.to(DEV).requires_grad_()
    out = m(xg)
    out.backward(gout.to(DEV))
    torch.cuda.synchronize()
    assert out.dtype == torch.float16 and out.shape == (N, C, H, H)

    # the module's own arithmetic up to the operator, restated on the CPU in float32
    wt = m.weight.detach().float().cpu()                # [C, 1, 5, 5], float16 values
    fw, fb = m.fc.weight.detach().float().cpu(), m.fc.bias.detach().float().cpu()
    centre = torch.tensor(m.fc_bias, dtype=torch.float32)
    pooled = x.float().mean((2, 3))
    coord_raw = pooled @ fw.t() + fb + centre
    coord = coord_raw.clamp(0, 4)
    open_ = ((coord_raw >= 0) & (coord_raw <= 4)).float()
    assert 0.005 < 1 - open_.mean().item() < 0.6        # the clamp to the scope is active on some taps
    rot_img = coord - centre                            # [N, 18]
    cfg = dict(kernel_size=(3, 3), stride=(1, 1), padding=(1, 1), dilation=(1, 1), groups=1)
    rot_full = rot_img.view(N, 18, 1, 1).expand(N, 18, H, H).contiguous()
    f = lambda t: t.float().numpy()
    gin, grot, gw = orc.sample_depthwise_backward(f(gout), f(x), f(rot_full), f(wt), **cfg)
    g_coord = torch.as_tensor(grot).sum((2, 3)) * open_  # [N, 18], through the clamp
    for n in (0, 77):
        sl = slice(n, n + 1)
        want = orc.sample_depthwise_forward(f(x[sl]), f(rot_full[sl]), f(wt), **cfg)
        _within(rel_err(out[sl].detach().float().cpu(), want), 1e-2, ("forward", n))
        # the input also feeds the pooled branch: mean over the plane -> fc -> offsets
        gx = torch.as_tensor(gin[sl]) + ((g_coord[sl] @ fw) / (H * H)).view(1, C, 1, 1)
        _within(rel_err(xg.grad[sl].float().cpu(), gx), 1e-2, ("grad input", n))
    _within(rel_err(m.weight.grad.float().cpu(), gw), 1e-2, "grad scope weight")
    _within(rel_err(m.fc.bias.grad.float().cpu(), g_coord.sum(0)), 2e-2, "grad fc bias")
    _within(rel_err(m.fc.weight.grad.float().cpu(), g_coord.t() @ pooled), 2e-2, "grad fc weight")

    # The reference's own route (nd_linear_sample + one convolution with N * C groups) on the same
    # module.  A float16 module evaluates the fc there in float16, as the reference does, and the
    # undeformed taps sit on integer scope coordinates: a coordinate that float16 rounds across a cell
    # border takes the next cell's slope, so the gradients that pass through the coordinates (fc.*, and a
    # constant per plane of the input gradient) jump for that tap -- inherent to that route, and left out
    # of the comparison: the input gradient is compared after removing each plane's mean.
    m.fused = False
    for p in m.parameters():
        p.grad = None
    x2 = x.to(DEV).requires_grad_()
    out2 = m(x2)
    out2.backward(gout.to(DEV))
    torch.cuda.synchronize()
    _within(rel_err(out2.detach().float().cpu(), out.detach().float().cpu()), 1e-2, "unfused forward")
    centred = lambda t: t.float().cpu() - t.float().cpu().mean((2, 3), keepdim=True)
    _within(rel_err(centred(x2.grad), centred(xg.grad)), 1e-2, "unfused grad input")
    _within(rel_err(m.weight.grad.float().cpu(), gw), 2e-2, "unfused grad scope weight")

    # That run applied the sampled kernels with the library's per-image depthwise convolution (the
    # default); the framework's convolution with N * C groups on the same sampled kernels must agree
    # with it in every result, the gradients that pass through the coordinates included.
    native = [out2.detach().float().cpu(), x2.grad.float().cpu()] + [p.grad.float().cpu() for p in m.parameters()]
    m.native_conv = False
    for p in m.parameters():
        p.grad = None
    x3 = x.to(DEV).requires_grad_()
    out3 = m(x3)
    out3.backward(gout.to(DEV))
    torch.cuda.synchronize()
    library = [out3.detach().float().cpu(), x3.grad.float().cpu()] + [p.grad.float().cpu() for p in m.parameters()]
    for name, a, b in zip(("forward", "grad input", "grad scope weight", "grad fc weight", "grad fc bias"), native, library):
        _within(rel_err(a, b), 1e-2, "per-image convolution against the framework's: " + name)


def test_config3_kernel_synthesis_float16():
    """The sampler call of configuration 3: 1152 = 128 x 9 points on 256 kernels of 5 x 5, float16."""
    from deformable_kernels.ops.deform_kernel.functions import nd_linear_sample
    g = torch.Generator().manual_seed(31)
    data = (torch.randn(256, 5, 5, generator=g) * 0.3).half()
    coord = (torch.rand(1152, 2, generator=g) * 4.0).half()
    gout = torch.randn(1152, 256, generator=g).half()
    dg, cg = data.to(DEV).requires_grad_(), coord.to(DEV).requires_grad_()
    out = nd_linear_sample(dg, cg)
    out.backward(gout.to(DEV))
    torch.cuda.synchronize()
    f = lambda t: t.float().numpy()
    want = orc.nd_linear_sample_forward(f(data), f(coord))
    gd, gc = orc.nd_linear_sample_backward(f(gout), f(data), f(coord))
    _within(rel_err(out.detach().float().cpu(), want), 1e-2, "")
    _within(rel_err(dg.grad.float().cpu(), gd), 1e-2, "")
    _within(rel_err(cg.grad.float().cpu(), gc), 1e-2, "")


@pytest.mark.parametrize("lo,hi", [(-1.0, 1.0), (-1.0, 32.0)])
def test_config5_trilinear_sampler_at_2_to_the_20_points(lo, hi):
    """data [64, 32, 32, 32] float32, 2^20 points: uniform in [-1, 1]^3 as the configuration writes it
    (every point in the 8 cells round the origin corner, half of them in the fade band) and uniform
    over the whole volume.  The oracle is run on a random subset of 8192 points (every point's output
    row and coordinate gradient depend on that point alone); the data gradient, a sum over all points,
    is checked through <gout, F(data)> = <grad_data, data> and, as F is linear in data, against the
    float64 oracle on a volume of which only one channel's gradient is taken."""
    from deformable_kernels.ops.deform_kernel.functions import nd_linear_sample
    B, C = 1 << 20, 64
    g = torch.Generator().manual_seed(50)
    data = torch.randn(C, 32, 32, 32, generator=g)
    coord = torch.rand(B, 3, generator=g) * (hi - lo) + lo
    gout = torch.randn(B, C, generator=g)
    dg, cg = data.to(DEV).requires_grad_(), coord.to(DEV).requires_grad_()
    out = nd_linear_sample(dg, cg)
    out.backward(gout.to(DEV))
    torch.cuda.synchronize()
    pick = torch.randperm(B, generator=g)[:8192]
    sub = coord[pick].contiguous()
    want = orc.nd_linear_sample_forward(data.numpy(), sub.numpy())
    _within(mixed_err(out.detach().cpu()[pick], want), 1e-5, "forward")
    _, gc = orc.nd_linear_sample_backward(gout[pick].double().numpy(), data.double().numpy(), sub.double().numpy())
    _within(rel_err(cg.grad.cpu()[pick], gc), 1e-4, "grad coord")
    # adjoint identity, sums in float64.  Both sides are sums of 2^26 signed terms of order 1 built from
    # float32 results (a spread of about 2^13 with a rounding error of about 2^13 * 2^-24 of it), and the
    # data gradient's float32 atomics add in an order that changes from run to run: 1e-5 of the larger side.
    a = (gout.to(DEV).double() * out.detach().double()).sum().item()
    b = (dg.grad.double() * dg.detach().double()).sum().item()
    assert abs(a - b) < 1e-5 * max(abs(a), abs(b), 1.0), (a, b)
    # one channel of the data gradient against the float64 oracle over all 2^20 points
    gd, _ = orc.nd_linear_sample_backward(gout[:, 5:6].double().numpy(), data[5:6].double().numpy(),
                                          coord.double().numpy())
    _within(rel_err(dg.grad[5:6].cpu(), gd), 1e-4, "grad data")


def _capture(layer, store):
    def hook(mod, inputs, output):
        store["x"], store["rot"] = inputs[0].detach(), inputs[1].detach()
        store["out"] = output.detach()
        output.register_hook(lambda g: store.__setitem__("gout", g.detach()))
    return layer.inner_conv.register_forward_hook(hook)


def test_config5_mobilenetv2_dk_network_bfloat16():
    """MobileNetV2 with its 17 depthwise 3 x 3 convolutions replaced by DeformKernel2d (scope 4 x 4),
    bfloat16 activations and parameters; the operator keeps float32 sums for the filter gradient.
    Batch 128: one forward + backward, every gradient finite and every deformable layer trained.
    Batch 2: the operator calls of all 17 layers as the network issues them (captured inputs, rotations
    and upstream gradients) against the float32 oracle on the same rounded tensors: forward and filter gradient."""
    from _mbv2_dk import MobileNetV2DK
    torch.manual_seed(5)
    net = MobileNetV2DK().to(DEV).to(torch.bfloat16)
    layers = net.dk_layers()
    assert len(layers) == 17
    assert [l.in_planes for l in layers] == [32, 96, 144, 144, 192, 192, 192, 384, 384, 384, 384, 576, 576, 576, 960, 960, 960]

    g = torch.Generator().manual_seed(51)
    x = torch.randn(128, 3, 224, 224, generator=g).to(DEV).to(torch.bfloat16)
    labels = torch.randint(0, 1000, (128,), generator=g).to(DEV)
    loss = torch.nn.functional.cross_entropy(net(x).float(), labels)
    loss.backward()
    torch.cuda.synchronize()
    assert torch.isfinite(loss).item()
    for name, p in net.named_parameters():
        assert p.grad is not None and bool(torch.isfinite(p.grad).all()), name
    for i, l in enumerate(layers):
        assert float(l.inner_conv.weight.grad.float().abs().max()) > 0, i
        assert float(l.rotation_conv.weight.grad.float().abs().max()) > 0, i

    # batch 2: every layer's operator calls against the oracle (112 x 112 C=32 down to 7 x 7 C=960, four of them stride 2)
    net.zero_grad(set_to_none=True)
    picked = {i: {} for i in range(17)}
    handles = [_capture(layers[i], st) for i, st in picked.items()]
    loss = torch.nn.functional.cross_entropy(net(x[:2]).float(), labels[:2])
    loss.backward()
    torch.cuda.synchronize()
    for h in handles:
        h.remove()
    f = lambda t: t.float().cpu().numpy()
    for i, st in picked.items():
        l = layers[i]
        cfg = dict(kernel_size=(3, 3), stride=(l.stride, l.stride), padding=(1, 1), dilation=(1, 1), groups=1)
        wt = l.inner_conv.weight.detach()
        assert float(st["rot"].float().abs().max()) > 0.05   # the layer does deform its kernels
        want = orc.sample_depthwise_forward(f(st["x"]), f(st["rot"]), f(wt), **cfg)
        _within(rel_err(st["out"].float().cpu(), want), 1e-2, "layer %d forward" % i)
        _, _, gw = orc.sample_depthwise_backward(f(st["gout"]), f(st["x"]), f(st["rot"]), f(wt), **cfg)
        _within(rel_err(l.inner_conv.weight.grad.float().cpu(), gw), 1e-2, "layer %d grad filter" % i)
