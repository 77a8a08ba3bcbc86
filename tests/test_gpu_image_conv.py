"""The per-image depthwise convolution (the convolution GlobalDeformKernel2d applies with its sampled
kernels, reference modules/deform_kernel.py:103-111) through the C ABI against the CPU oracle:
float32 and float64 within 1e-5 (forward, input gradient) / 1e-4 (kernel gradient, a sum over the
plane) of the float64 oracle relative to the result's largest magnitude; float16 / bfloat16
within 1e-2 of the oracle evaluated on the rounded inputs."""
import ctypes

import numpy as np
import pytest
import torch

from _cases import rel_err
from oracle import dk_oracle as orc

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")

CASES = [
    # N, C, H, W, k_h, k_w, stride, padding, dilation
    (3, 10, 28, 28, 3, 3, (1, 1), (1, 1), (1, 1)),    # configuration 3's plane: one band, aligned rows
    (2, 5, 9, 7, 3, 3, (1, 1), (1, 1), (1, 1)),       # odd width: scalar stores, partial strips
    (2, 6, 56, 56, 3, 3, (1, 1), (1, 1), (1, 1)),     # two bands per plane
    (1, 3, 112, 112, 3, 3, (1, 1), (1, 1), (1, 1)),   # many bands, rows wider than a wave
    (2, 7, 28, 28, 3, 3, (2, 2), (1, 1), (1, 1)),     # stride 2: strided input gradient
    (2, 4, 15, 22, 3, 3, (2, 1), (0, 2), (1, 2)),     # mixed strides, dilation, no padding in h
    (1, 5, 17, 13, 3, 3, (1, 1), (2, 2), (2, 2)),     # dilation 2 at stride 1: flipped-tap input gradient
    (2, 3, 14, 14, 5, 5, (1, 1), (2, 2), (1, 1)),     # 5 x 5 taps
    (2, 3, 12, 10, 1, 1, (1, 1), (0, 0), (1, 1)),     # 1 x 1 taps
    (1, 4, 13, 9, 3, 2, (1, 1), (1, 0), (1, 1)),      # run-time tap counts
    (1, 2, 20, 16, 7, 7, (2, 2), (3, 3), (1, 1)),     # run-time tap counts, strided
    (1, 3, 6, 6, 3, 3, (1, 1), (3, 3), (1, 1)),       # padding wider than the kernel's reach
    (5, 1, 8, 8, 3, 3, (1, 1), (1, 1), (1, 1)),       # planes not a multiple of the waves per workgroup
]


def _run(case, dtype, seed=0, sampler_layout=False):
    """sampler_layout: the kernels as the N-d sampler leaves them, [N * k_h * k_w, C], handed over as
    a permuted [N, C, k_h, k_w] view (element strides instead of a transposing copy)."""
    from deformable_kernels.ops.deform_kernel.functions import image_depthwise_conv, image_depthwise_conv_supported
    N, C, H, W, kh, kw, stride, pad, dil = case
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(N, C, H, W, generator=g, dtype=torch.float64).to(dtype)
    w = torch.randn(N * C, 1, kh, kw, generator=g, dtype=torch.float64).to(dtype)
    xg = x.to(DEV).requires_grad_()
    if sampler_layout:
        leaf = w.view(N, C, kh, kw).permute(0, 2, 3, 1).contiguous().view(N * kh * kw, C).to(DEV).requires_grad_()
        wg = leaf.view(N, kh, kw, C).permute(0, 3, 1, 2)
        assert C == 1 or not wg.is_contiguous()
    else:
        leaf = wg = w.to(DEV).requires_grad_()
    assert image_depthwise_conv_supported(xg, wg, stride, pad, dil)
    out = image_depthwise_conv(xg, wg, stride, pad, dil)
    gout = torch.randn(out.shape, generator=g, dtype=torch.float64).to(dtype)
    out.backward(gout.to(DEV))
    torch.cuda.synchronize()
    gw_got = leaf.grad.cpu()
    gw_got = gw_got.view(N, kh, kw, C).permute(0, 3, 1, 2) if sampler_layout else gw_got.view(N, C, kh, kw)
    x64, w64, g64 = x.double().numpy(), w.double().view(N, C, kh, kw).numpy(), gout.double().numpy()
    want = orc.image_depthwise_forward(x64, w64, stride, pad, dil)
    gx, gw = orc.image_depthwise_backward(g64, x64, w64, stride, pad, dil)
    return (out.detach().cpu(), xg.grad.cpu(), gw_got), (want, gx, gw)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("case", CASES)
def test_full_precision_against_the_float64_oracle(case, dtype):
    got, want = _run(case, dtype)
    assert got[0].dtype == dtype and got[0].shape == want[0].shape
    assert rel_err(got[0], want[0]) < 1e-5
    assert rel_err(got[1], want[1]) < 1e-5
    assert rel_err(got[2], want[2]) < 1e-4


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("case", CASES[:5] + CASES[9:10] + CASES[12:])
def test_kernels_in_the_layout_the_sampler_leaves_them(case, dtype):
    got, want = _run(case, dtype, seed=2, sampler_layout=True)
    tol = (1e-5, 1e-5, 1e-4) if dtype == torch.float32 else (1e-2, 1e-2, 1e-2)
    for a, b, t in zip(got, want, tol):
        assert rel_err(a.float(), b) < t


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", CASES[:4] + CASES[12:])
def test_band_kernels_on_the_shapes_the_flat_copy_kernels_serve(case, dtype, switch_off):
    """3 x 3 taps, stride 1, padding 1 go to the kernels that stage a band as a flat copy; with that
    family switched off the general band kernels serve the same shapes."""
    switch_off("DK_NO_IMAGE_FLAT")
    got, want = _run(case, dtype, seed=3, sampler_layout=case[1] % 2 == 0)
    tol = (1e-5, 1e-5, 1e-4) if dtype == torch.float32 else (1e-2, 1e-2, 1e-2)
    for a, b, t in zip(got, want, tol):
        assert rel_err(a.float(), b) < t


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", CASES[:6] + CASES[9:10])
def test_16_bit_types_against_the_oracle_on_the_rounded_inputs(case, dtype):
    got, want = _run(case, dtype, seed=5)
    for a, b in zip(got, want):
        assert a.dtype == dtype
        assert rel_err(a.float(), b) < 1e-2


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", [CASES[0], CASES[2], CASES[3], CASES[12]])
def test_packed_16_bit_kernels_against_the_kernels_that_unpack(case, dtype, switch_off):
    """16-bit tensors with rows of a multiple of 4 elements stay packed in LDS and are summed two products per
    instruction (fp32 sums); switched off, the flat-copy kernels that unpack to fp32 serve the shapes.  Both
    sum in fp32 and round once, so they differ by the result's last bit at most, and both meet the oracle."""
    got, want = _run(case, dtype, seed=11)
    switch_off("DK_NO_IMAGE_PACKED")
    got2, _ = _run(case, dtype, seed=11)
    ulp = 2.0 ** -10 if dtype == torch.float16 else 2.0 ** -7
    for a, b, w in zip(got, got2, want):
        assert rel_err(a.float(), w) < 1e-2 and rel_err(b.float(), w) < 1e-2
        assert ((a.float() - b.float()).abs() <= ulp * b.float().abs() + 1e-6 * b.float().abs().max()).all()


def _packed_cases():
    import random
    rnd = random.Random(41)
    return [(rnd.choice([1, 2, 5]), rnd.choice([1, 3, 4, 9]), rnd.choice([1, 2, 3, 4, 5, 8, 12, 17, 40, 64]),
             rnd.choice([4, 8, 12, 20, 36, 60, 100, 128]), 3, 3, (1, 1), (1, 1), (1, 1)) for _ in range(14)]


@pytest.mark.parametrize("k,case", list(enumerate(_packed_cases())))
def test_packed_16_bit_kernels_on_random_planes(k, case):
    """Rows of 4 to 128 elements, planes of one row to several bands, plane counts that fill no workgroup."""
    dtype = torch.float16 if k % 2 == 0 else torch.bfloat16
    got, want = _run(case, dtype, seed=20 + k, sampler_layout=k % 3 == 0)
    for a, b in zip(got, want):
        assert a.dtype == dtype
        assert rel_err(a.float(), b) < 1e-2


def test_configuration_3_shape_float16_matches_the_grouped_convolution_it_replaces():
    """N=128, C=256, 28x28, 3x3 kernels per (image, channel), float16: the oracle on three images, and
    the framework's convolution with N * C groups (the reference's call) on the whole batch."""
    from deformable_kernels.ops.deform_kernel.functions import image_depthwise_conv
    N, C, H = 128, 256, 28
    g = torch.Generator().manual_seed(8)
    x = torch.randn(N, C, H, H, generator=g).half()
    w = (torch.randn(N * C, 1, 3, 3, generator=g) * 0.3).half()
    gout = torch.randn(N, C, H, H, generator=g).half()
    xg, wg = x.to(DEV).requires_grad_(), w.to(DEV).requires_grad_()
    out = image_depthwise_conv(xg, wg, 1, 1, 1)
    out.backward(gout.to(DEV))
    x2, w2 = x.to(DEV).requires_grad_(), w.to(DEV).requires_grad_()
    ref = torch.nn.functional.conv2d(x2.view(1, N * C, H, H), w2, padding=1, groups=N * C).view(N, C, H, H)
    ref.backward(gout.to(DEV))
    torch.cuda.synchronize()
    assert rel_err(out.float().cpu(), ref.float().cpu()) < 1e-2
    assert rel_err(xg.grad.float().cpu(), x2.grad.float().cpu()) < 1e-2
    assert rel_err(wg.grad.float().cpu(), w2.grad.float().cpu()) < 1e-2
    for n in (0, 64, 127):
        sl = slice(n, n + 1)
        x64, g64 = x[sl].double().numpy(), gout[sl].double().numpy()
        w64 = w.view(N, C, 3, 3)[sl].double().numpy()
        assert rel_err(out[sl].float().cpu(), orc.image_depthwise_forward(x64, w64, 1, 1, 1)) < 1e-2
        gx, gw = orc.image_depthwise_backward(g64, x64, w64, 1, 1, 1)
        assert rel_err(xg.grad[sl].float().cpu(), gx) < 1e-2
        assert rel_err(wg.grad.view(N, C, 3, 3)[sl].float().cpu(), gw) < 1e-2


def test_c_abi_rejections_and_empty_batch():
    from deformable_kernels.ops.deform_kernel import _lib
    L = _lib.lib()
    x = torch.zeros(1, 2, 8, 8, device=DEV)
    w = torch.zeros(2, 1, 3, 3, device=DEV)
    out = torch.zeros(1, 2, 8, 8, device=DEV)
    desc = _lib.ConvDesc(1, 2, 8, 8, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, _lib.DK_F32, 0, 0.0, 0.0)
    st = _lib.stream_ptr(x)
    assert L.dk_image_depthwise_forward(desc, None, _lib.ptr(w), None, _lib.ptr(out), st) == -1  # DK_ERR_NULL_POINTER
    negative = (ctypes.c_int64 * 4)(18, 9, -3, 1)
    assert L.dk_image_depthwise_forward(desc, _lib.ptr(x), _lib.ptr(w), negative, _lib.ptr(out), st) == -2  # DK_ERR_BAD_SHAPE
    # a row of taps that does not fit a wave's staging area: refused, the caller keeps its own convolution
    wide = _lib.ConvDesc(1, 2, 8, 4000, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, _lib.DK_F32, 0, 0.0, 0.0)
    assert L.dk_image_depthwise_supported(wide) == 0
    assert L.dk_image_depthwise_forward(wide, _lib.ptr(x), _lib.ptr(w), None, _lib.ptr(out), st) == -7  # DK_ERR_UNSUPPORTED
    empty = _lib.ConvDesc(0, 2, 8, 8, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, _lib.DK_F32, 0, 0.0, 0.0)
    assert L.dk_image_depthwise_forward(empty, _lib.ptr(x), _lib.ptr(w), None, _lib.ptr(out), st) == 0
    assert L.dk_image_depthwise_backward_data(empty, _lib.ptr(out), _lib.ptr(w), None, _lib.ptr(x), st) == 0
    assert L.dk_image_depthwise_backward_weight(empty, _lib.ptr(out), _lib.ptr(x), _lib.ptr(w), None, st) == 0
    torch.cuda.synchronize()
