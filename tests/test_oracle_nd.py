"""Pins the oracle's N-d linear sampler: numpy.interp (n = 1), grid_sample
4-D / 5-D with autograd (n = 2, 3), the hat-function tensor product for
n = 4, the zero rule at x <= -1 and x >= s, and the border fade bands."""
import itertools

import numpy as np
import pytest
import torch

import _composite as comp
from _cases import rel_err
from oracle import dk_oracle as orc


def _hat(t):
    return np.maximum(0.0, 1.0 - np.abs(t))


def test_one_dimension_matches_numpy_interp_inside_the_range():
    rng = np.random.default_rng(31)
    data = rng.standard_normal((5, 9))
    coord = rng.uniform(0, 8, size=(40, 1))
    got = orc.nd_linear_sample_forward(data, coord)
    want = np.stack([np.interp(coord[:, 0], np.arange(9), data[c]) for c in range(5)], 1)
    assert rel_err(got, want) < 1e-14


@pytest.mark.parametrize("shape", [(6, 5), (4, 5, 6)])
def test_forward_and_gradients_match_grid_sample(shape):
    g = torch.Generator().manual_seed(32)
    C, B = 7, 64
    data = torch.randn(C, *shape, generator=g, dtype=torch.float64)
    hi = torch.tensor(shape, dtype=torch.float64)
    coord = torch.rand(B, len(shape), generator=g, dtype=torch.float64) * (hi + 3) - 2  # spills outside
    gout = torch.randn(B, C, generator=g, dtype=torch.float64)
    dr, cr = data.clone().requires_grad_(), coord.clone().requires_grad_()
    want = comp.nd_sample(dr, cr)
    want.backward(gout)
    got = orc.nd_linear_sample_forward(data.numpy(), coord.numpy())
    assert rel_err(got, want.detach()) < 1e-13
    gdata, gcoord = orc.nd_linear_sample_backward(gout.numpy(), data.numpy(), coord.numpy())
    assert rel_err(gdata, dr.grad) < 1e-13
    assert rel_err(gcoord, cr.grad) < 1e-13


def test_four_dimensions_match_hat_function_tensor_product():
    rng = np.random.default_rng(33)
    shape = (3, 4, 2, 5)
    data = rng.standard_normal((2,) + shape)
    coord = rng.uniform(-1.5, 5.5, size=(50, 4))
    coord[0] = [0, 0, 0, 0]
    coord[1] = [2, 3, 1, 4]          # last cell exactly
    coord[2] = [-0.5, 3.5, 1.25, 4.5]  # fade bands
    got = orc.nd_linear_sample_forward(data, coord)
    want = np.zeros_like(got)
    for b in range(coord.shape[0]):
        inside = all(-1 < coord[b, d] < shape[d] for d in range(4))
        if not inside:
            continue
        wts = [_hat(coord[b, d] - np.arange(shape[d])) for d in range(4)]
        for idx in itertools.product(*[range(s) for s in shape]):
            wgt = np.prod([wts[d][idx[d]] for d in range(4)])
            if wgt:
                want[b] += wgt * data[(slice(None),) + idx]
    assert rel_err(got, want) < 1e-13


def test_zero_rule_is_closed_at_minus_one_and_at_size():
    data = np.ones((1, 4, 4))
    pts = np.array([[-1.0, 1.0], [1.0, -1.0], [4.0, 1.0], [1.0, 4.0], [-0.5, 1.0], [3.5, 3.5], [3.0, 3.0]])
    got = orc.nd_linear_sample_forward(data, pts)[:, 0]
    assert list(got[:4]) == [0, 0, 0, 0]
    assert np.allclose(got[4:], [0.5, 0.25, 1.0])
    gdata, gcoord = orc.nd_linear_sample_backward(np.ones((7, 1)), data, pts)
    assert np.count_nonzero(gcoord[:4]) == 0


def test_coordinate_gradient_is_the_derivative_of_forward():
    rng = np.random.default_rng(34)
    data = rng.standard_normal((3, 4, 5, 3))
    coord = rng.uniform(-0.9, 3.9, size=(20, 3)) * np.array([1.0, 1.2, 0.7])
    fr = coord - np.floor(coord)
    coord += 0.01 * (np.minimum(fr, 1 - fr) < 1e-3)
    gout = rng.standard_normal((20, 3))
    gdata, gcoord = orc.nd_linear_sample_backward(gout, data, coord)
    eps = 1e-6
    for b in range(20):
        for d in range(3):
            cp, cm = coord.copy(), coord.copy()
            cp[b, d] += eps
            cm[b, d] -= eps
            num = ((orc.nd_linear_sample_forward(data, cp) - orc.nd_linear_sample_forward(data, cm)) * gout).sum() / (2 * eps)
            assert abs(num - gcoord[b, d]) < 1e-6 * max(1.0, abs(num))
    # grad_data is the adjoint of the (linear in data) forward map
    probe = rng.standard_normal(data.shape)
    lhs = (orc.nd_linear_sample_forward(probe, coord) * gout).sum()
    assert abs(lhs - (probe * gdata).sum()) < 1e-10 * max(1.0, abs(lhs))


def test_float32_tracks_float64():
    rng = np.random.default_rng(35)
    data = rng.standard_normal((8, 5, 5))
    coord = rng.uniform(-1.2, 5.2, size=(100, 2))
    gout = rng.standard_normal((100, 8))
    a = orc.nd_linear_sample_forward(data.astype(np.float32), coord.astype(np.float32))
    assert a.dtype == np.float32
    assert rel_err(a, orc.nd_linear_sample_forward(data, coord)) < 1e-5
