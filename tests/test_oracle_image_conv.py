"""CPU tests that pin the oracle's per-image depthwise convolution (the convolution
GlobalDeformKernel2d applies with its sampled kernels, reference modules/deform_kernel.py:103-111)
against the routine the reference calls there: torch's conv2d with n * c groups on
x.view(1, n * c, h, w), and the gradients its autograd derives, in float64."""
import numpy as np
import pytest
import torch

from oracle import dk_oracle as orc

CASES = [
    # N, C, H, W, k_h, k_w, stride, padding, dilation
    (2, 3, 9, 8, 3, 3, (1, 1), (1, 1), (1, 1)),
    (2, 3, 9, 8, 3, 3, (2, 2), (1, 1), (1, 1)),
    (1, 4, 11, 7, 3, 3, (2, 1), (0, 2), (1, 2)),
    (2, 2, 10, 10, 5, 5, (1, 1), (2, 2), (1, 1)),
    (1, 3, 12, 9, 3, 2, (3, 2), (2, 0), (2, 1)),
    (2, 2, 6, 6, 1, 1, (1, 1), (0, 0), (1, 1)),
    (1, 2, 5, 5, 3, 3, (1, 1), (3, 3), (1, 1)),  # padding wider than the kernel's reach
]


def _inputs(case, seed=0):
    N, C, H, W, kh, kw, stride, pad, dil = case
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(N, C, H, W, generator=g, dtype=torch.float64)
    w = torch.randn(N, C, kh, kw, generator=g, dtype=torch.float64)
    return x, w


def _torch_route(x, w, stride, pad, dil):
    """The reference's call: one convolution with n * c groups."""
    N, C, H, W = x.shape
    out = torch.nn.functional.conv2d(x.reshape(1, N * C, H, W), w.reshape(N * C, 1, *w.shape[2:]),
                                     stride=stride, padding=pad, dilation=dil, groups=N * C)
    return out.view(N, C, out.shape[2], out.shape[3])


@pytest.mark.parametrize("case", CASES)
def test_forward_and_gradients_match_grouped_conv2d(case):
    stride, pad, dil = case[6:]
    x, w = _inputs(case)
    xt, wt = x.clone().requires_grad_(), w.clone().requires_grad_()
    want = _torch_route(xt, wt, stride, pad, dil)
    gout = torch.randn(want.shape, generator=torch.Generator().manual_seed(1), dtype=torch.float64)
    want.backward(gout)
    got = orc.image_depthwise_forward(x.numpy(), w.numpy(), stride, pad, dil)
    assert got.shape == tuple(want.shape)
    np.testing.assert_allclose(got, want.detach().numpy(), rtol=1e-12, atol=1e-12)
    gx, gw = orc.image_depthwise_backward(gout.numpy(), x.numpy(), w.numpy(), stride, pad, dil)
    np.testing.assert_allclose(gx, xt.grad.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(gw, wt.grad.numpy(), rtol=1e-12, atol=1e-12)


def test_single_tap_kernel_picks_the_shifted_plane():
    """A kernel that is 1 at tap (i, j) and 0 elsewhere returns the zero-padded plane shifted by that
    tap: fixes the tap order (row-major, cross-correlation: no flip) and the zero border."""
    x = np.arange(2 * 1 * 4 * 5, dtype=np.float64).reshape(2, 1, 4, 5) + 1
    for i in range(3):
        for j in range(3):
            w = np.zeros((2, 1, 3, 3))
            w[:, :, i, j] = 1.0
            y = orc.image_depthwise_forward(x, w, (1, 1), (1, 1), (1, 1))
            xp = np.pad(x, ((0, 0), (0, 0), (1, 1), (1, 1)))
            np.testing.assert_array_equal(y, xp[:, :, i:i + 4, j:j + 5])
