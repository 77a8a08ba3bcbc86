"""The offset branch's 3x3 convolution (the library's kernels for LocalDeformKernel2d's
rotation_conv) against the float64 convolution computed on the CPU: every pass within 1e-5 of it
(relative to its largest magnitude) for float32 tensors -- as bfloat16 pairs on the 16-bit matrix
instructions, and with that switched off as the fp32 matrix-instruction forward -- within the
results' own rounding for 16-bit tensors, and the module with the kernels switched on and off."""
import contextlib

import pytest
import torch
import torch.nn.functional as F

from _cases import rel_err

pytestmark = pytest.mark.gpu


def reference(x, w, b, gout=None, stride=1):
    """float64 convolution on the CPU of the tensors' values: out (and gx, gw, gb for a gout, which may be a
    function of the output's shape)."""
    xd, wd, bd = [t.detach().cpu().double().requires_grad_() for t in (x, w, b)]
    out = F.conv2d(xd, wd, bd, stride=stride, padding=1)
    if gout is None:
        return out.detach()
    out.backward(gout.detach().cpu().double())
    return out.detach(), xd.grad, wd.grad, bd.grad


def switches(pairs):
    from deformable_kernels.ops.deform_kernel import _lib
    return contextlib.nullcontext() if pairs else _lib.test_switches("DK_NO_OFFSET_PAIRS")


@pytest.mark.parametrize("shape", [
    (2, 16, 5, 7, 18),      # N, C, H, W, out channels: one partial tile
    (3, 32, 14, 14, 18),
    (2, 48, 28, 28, 18),    # tile rows 8: the last tile has 4 rows
    (2, 144, 56, 56, 18),   # the headline layer's offset branch
    (1, 32, 9, 112, 18),    # two 64-column segments per staged row, tile rows 4
    (2, 32, 56, 56, 16),    # no outputs beyond the matrix-core tile
    (2, 32, 20, 56, 8),     # fewer than 16 outputs
    (1, 16, 13, 28, 20),    # four outputs on the vector path
])
@pytest.mark.parametrize("pairs", [True, False])
def test_forward_matches_float64_convolution(shape, pairs):
    from deformable_kernels.ops.deform_kernel.functions import offset_conv, offset_conv_supported
    N, C, H, W, O = shape
    g = torch.Generator().manual_seed(31)
    dev = torch.device("cuda:0")
    x = torch.randn(N, C, H, W, generator=g).to(dev)
    w = (torch.randn(O, C, 3, 3, generator=g) * 0.05).to(dev)
    b = torch.randn(O, generator=g).to(dev)
    with switches(pairs):
        assert offset_conv_supported(x, w, b, 1, 1, 1)
        got = offset_conv(x, w, b, force=True)
    want = reference(x, w, b)
    assert got.shape == want.shape and got.dtype == torch.float32
    assert rel_err(got.cpu(), want) < 1e-5


@pytest.mark.parametrize("shape", [
    (2, 16, 5, 7, 18), (3, 32, 14, 14, 18), (2, 48, 28, 28, 18), (2, 144, 56, 56, 18), (1, 32, 9, 112, 18),
    (2, 32, 56, 56, 16), (1, 16, 13, 28, 20), (40, 32, 56, 56, 18),   # the last: several items per workgroup
])
@pytest.mark.parametrize("pairs", [True, False])   # False: the fp32 matrix-instruction weight gradient as well
def test_gradients_match_float64(shape, pairs):
    """float32 tensors: input gradient on the bfloat16-pair kernel (the framework's with the pairs off), weight
    gradient on the fp32 matrix instructions, bias gradient by the library's reduction."""
    from deformable_kernels.ops.deform_kernel.functions import offset_conv
    N, C, H, W, O = shape
    g = torch.Generator().manual_seed(33)
    dev = torch.device("cuda:0")
    x = torch.randn(N, C, H, W, generator=g).to(dev).requires_grad_()
    w = (torch.randn(O, C, 3, 3, generator=g) * 0.05).to(dev).requires_grad_()
    b = torch.randn(O, generator=g).to(dev).requires_grad_()
    gout = torch.randn(N, O, H, W, generator=g).to(dev)
    with switches(pairs):
        offset_conv(x, w, b, force=True).backward(gout)
    _, gx, gw, gb = reference(x, w, b, gout)
    assert rel_err(w.grad.cpu(), gw) < 1e-5
    assert rel_err(b.grad.cpu(), gb) < 1e-5
    assert rel_err(x.grad.cpu(), gx) < 1e-5


@pytest.mark.parametrize("dtype,tol", [(torch.float16, 2e-3), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("shape", [(2, 16, 5, 7, 18), (3, 32, 14, 14, 18), (2, 144, 56, 56, 18), (1, 32, 9, 112, 18),
                                   (2, 32, 56, 56, 16), (40, 32, 56, 56, 18), (64, 960, 7, 7, 18),
                                   (3, 192, 28, 28, 18), (2, 48, 13, 28, 18), (1, 16, 3, 56, 18), (2, 80, 21, 112, 20)])
def test_sixteen_bit_tensors_match_float64_on_the_rounded_inputs(shape, dtype, tol):
    """float16 / bfloat16 tensors: fp32 sums of exact products everywhere, so the error against the float64
    convolution of the rounded inputs is the results' own rounding.  Planes 28, 56 and 112 wide take the forward
    and the input gradient on the 16-bit matrix-instruction kernel (whole and partial row tiles, channel counts
    that leave half a chunk of 32, 16 / 18 / 20 outputs), the others the fp32-arithmetic forward and the
    library's input gradient; weight and bias gradient have fp32 partial sums."""
    from deformable_kernels.ops.deform_kernel.functions import offset_conv, offset_conv_supported
    N, C, H, W, O = shape
    g = torch.Generator().manual_seed(37)
    dev = torch.device("cuda:0")
    x = torch.randn(N, C, H, W, generator=g).to(dtype).to(dev).requires_grad_()
    w = (torch.randn(O, C, 3, 3, generator=g) * 0.05).to(dtype).to(dev).requires_grad_()
    b = torch.randn(O, generator=g).to(dtype).to(dev).requires_grad_()
    gout = torch.randn(N, O, H, W, generator=g).to(dtype).to(dev)
    assert offset_conv_supported(x, w, b, 1, 1, 1)
    out = offset_conv(x, w, b, force=True)
    assert out.dtype == dtype
    out.backward(gout)
    want, gx, gw, gb = reference(x, w, b, gout)
    assert rel_err(out.detach().double().cpu(), want) < tol
    assert w.grad.dtype == dtype and b.grad.dtype == dtype
    assert rel_err(w.grad.double().cpu(), gw) < tol
    assert rel_err(b.grad.double().cpu(), gb) < tol
    assert x.grad.dtype == dtype
    assert rel_err(x.grad.double().cpu(), gx) < tol


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.float16, 2e-3), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("shape", [(2, 96, 112, 112, 18), (3, 144, 56, 56, 18), (2, 192, 28, 28, 18), (5, 576, 14, 14, 18),
                                   (2, 32, 9, 56, 18), (1, 16, 1, 14, 16), (2, 48, 30, 28, 20), (2, 32, 17, 112, 7)])
def test_stride_2_forward_and_input_gradient(shape, dtype, tol):
    """The down-sampling layers' convolution (stride 2, padding 1): forward and input gradient on the 16-bit matrix
    instructions -- float16 / bfloat16 elements as they are, float32 ones as bfloat16 pairs (two chunks of output
    gradient channels in the input gradient) -- over whole, partial and single-row tiles, odd heights, half
    chunks of channels, planes lower than a tile, chunk splits, one to three blocks of 16 channels; the weight
    gradient on the framework's routine, the bias gradient on the library's."""
    from deformable_kernels.ops.deform_kernel.functions import offset_conv, offset_conv_supported
    N, C, H, W, O = shape
    g = torch.Generator().manual_seed(43)
    dev = torch.device("cuda:0")
    x = torch.randn(N, C, H, W, generator=g).to(dtype).to(dev).requires_grad_()
    w = (torch.randn(O, C, 3, 3, generator=g) * 0.05).to(dtype).to(dev).requires_grad_()
    b = torch.randn(O, generator=g).to(dtype).to(dev).requires_grad_()
    assert offset_conv_supported(x, w, b, 2, 1, 1)
    if dtype == torch.float32:
        with switches(False):
            assert not offset_conv_supported(x, w, b, 2, 1, 1)
    out = offset_conv(x, w, b, stride=2, force=True)
    gout = torch.randn(out.shape, generator=g).to(dtype).to(dev)
    want, gx, gw, gb = reference(x, w, b, gout, stride=2)
    assert out.shape == want.shape and out.dtype == dtype
    assert rel_err(out.detach().double().cpu(), want) < tol
    out.backward(gout)
    assert rel_err(x.grad.double().cpu(), gx) < tol
    assert rel_err(w.grad.double().cpu(), gw) < tol
    assert rel_err(b.grad.double().cpu(), gb) < tol


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("wgrad16", [True, False])
def test_fewer_than_15_outputs(dtype, tol, wgrad16):
    """Seven outputs: every pass has a kernel on the 16-bit matrix instructions; with that weight gradient switched
    off the fp32 matrix-instruction one, which covers 15 and more outputs, answers its workspace query with 0 and
    the weight gradient comes from the framework's routine."""
    from deformable_kernels.ops.deform_kernel.functions import offset_conv, offset_conv_supported
    g = torch.Generator().manual_seed(41)
    dev = torch.device("cuda:0")
    x = torch.randn(2, 32, 9, 56, generator=g).to(dtype).to(dev).requires_grad_()
    w = (torch.randn(7, 32, 3, 3, generator=g) * 0.05).to(dtype).to(dev).requires_grad_()
    b = torch.randn(7, generator=g).to(dtype).to(dev).requires_grad_()
    gout = torch.randn(2, 7, 9, 56, generator=g).to(dtype).to(dev)
    from deformable_kernels.ops.deform_kernel import _lib
    with contextlib.nullcontext() if wgrad16 else _lib.test_switches("DK_NO_OFFSET_WGRAD16"):
        assert offset_conv_supported(x, w, b, 1, 1, 1)
        assert (_lib.lib().dk_offset_conv_backward_weight_workspace(
            _lib.OffsetConvDesc(2, 32, 7, 9, 56, _lib.dtype_tag(x), 1)) > 0) == wgrad16
        out = offset_conv(x, w, b, force=True)
        out.backward(gout)
    want, gx, gw, gb = reference(x, w, b, gout)
    for got, ref in ((out.detach(), want), (x.grad, gx), (w.grad, gw), (b.grad, gb)):
        assert got.dtype == dtype and rel_err(got.double().cpu(), ref) < tol


def test_unsupported_calls_go_to_the_library_convolution():
    from deformable_kernels.ops.deform_kernel.functions import offset_conv, offset_conv_supported
    dev = torch.device("cuda:0")
    x = torch.randn(2, 24, 10, 10, device=dev)   # 24 channels: not a multiple of 16; width 10
    w = torch.randn(18, 24, 3, 3, device=dev)
    assert not offset_conv_supported(x, w, None, 1, 1, 1)
    assert torch.equal(offset_conv(x, w, None), F.conv2d(x, w, None, 1, 1, 1))
    x2 = torch.randn(2, 32, 56, 56, device=dev)
    w2 = torch.randn(18, 32, 3, 3, device=dev)
    with switches(False):
        assert not offset_conv_supported(x2, w2, None, 2, 1, 1)      # stride 2, float32, without the pair kernels
    assert not offset_conv_supported(x2[:, :, :, :20].contiguous(), w2, None, 2, 1, 1)   # stride 2, 20 columns
    assert not offset_conv_supported(x2.double(), w2.double(), None, 1, 1, 1)   # float64
    assert not offset_conv_supported(x2.half(), w2, None, 1, 1, 1)              # mixed dtypes
    with switches(False):
        assert torch.equal(offset_conv(x2, w2, None, stride=2), F.conv2d(x2, w2, None, 2, 1, 1))
    assert torch.equal(offset_conv(x2.double(), w2.double(), None), F.conv2d(x2.double(), w2.double(), None, 1, 1, 1))


@pytest.mark.parametrize("conv", [(2, 1, 1), (1, 0, 1), (1, 2, 2), (2, 1, 1, 24)])
def test_other_convolutions_keep_the_library_kernels_but_not_its_bias_gradient(conv):
    # stride 2 / no padding / dilation 2 / 24 channels: the forward is F.conv2d's, the gradients match autograd's
    from deformable_kernels.ops.deform_kernel.functions import offset_conv
    stride, padding, dilation = conv[:3]
    C = conv[3] if len(conv) > 3 else 32
    g = torch.Generator().manual_seed(34)
    dev = torch.device("cuda:0")
    x = torch.randn(3, C, 20, 22, generator=g).to(dev).requires_grad_()
    w = (torch.randn(18, C, 3, 3, generator=g) * 0.05).to(dev).requires_grad_()
    b = torch.randn(18, generator=g).to(dev).requires_grad_()
    out = offset_conv(x, w, b, stride, padding, dilation)
    x2, w2, b2 = [t.detach().clone().requires_grad_() for t in (x, w, b)]
    ref = F.conv2d(x2, w2, b2, stride, padding, dilation)
    assert torch.equal(out, ref)
    gout = torch.randn(ref.shape, generator=g).to(dev)
    out.backward(gout)
    ref.backward(gout)
    assert rel_err(x.grad.cpu(), x2.grad.cpu()) < 1e-6
    assert rel_err(w.grad.cpu(), w2.grad.cpu()) < 1e-6
    assert rel_err(b.grad.cpu(), gout.double().sum((0, 2, 3)).float().cpu()) < 1e-5


def test_gradients_and_module_switch():
    from deformable_kernels.modules import LocalDeformKernel2d
    torch.manual_seed(32)
    dev = torch.device("cuda:0")
    C = 16
    m = LocalDeformKernel2d((4, 4), C, C, 3, 1, 1, 1, C, 1, False, 'scope').to(dev)
    torch.nn.init.normal_(m.rotation_conv.weight, std=0.1)
    x = torch.randn(28, C, 56, 56, device=dev)    # 28 images x 7 row tiles: the native kernel is chosen
    gout = torch.randn(28, C, 56, 56, device=dev)
    results = []
    for native, pairs in ((False, True), (True, True), (True, False)):
        m.native_offset_conv = native
        m.zero_grad()
        xi = x.clone().requires_grad_()
        with switches(pairs):
            out = m(xi)
            out.backward(gout)
        results.append([t.detach().cpu().clone() for t in (
            out, xi.grad, m.inner_conv.weight.grad, m.rotation_conv.weight.grad, m.rotation_conv.bias.grad)])
    # The branch's float32 kernels multiply bfloat16 pairs (3.5e-6 of the rotations' scale) and the operator's
    # output moves with its rotations: 1.7e-5 of the output's scale was measured here.  Its rotation gradient is
    # piecewise constant in the rotation (the slope of the bilinear patch): a rotation within that distance of a
    # cell border lands in the neighbouring cell and moves one element of the rotation gradient -- and the 144
    # input-gradient elements under it -- by a finite amount.  About ten of the 1.6 M coordinates do, so the
    # gradients are compared in the root mean square and by the share of elements that moved at all; with the
    # pairs switched off (5e-7) none flips and the element-wise bound holds.
    assert rel_err(results[1][0], results[0][0]) < 5e-5
    for got, ref in zip(results[1][1:], results[0][1:]):
        diff = (got - ref).abs()
        assert float(diff.pow(2).mean().sqrt() / ref.pow(2).mean().sqrt()) < 1e-2   # (2.2e-3 measured)
        if got.numel() > 100000:   # the input gradient: few elements move at all (the others are sums over pixels)
            assert float((diff > 1e-4 * ref.abs().max()).float().mean()) < 5e-3
    assert rel_err(results[2][0], results[0][0]) < 1e-5
    for got, ref in zip(results[2][1:], results[0][1:]):
        assert rel_err(got, ref) < 1e-4
