"""Pins the CPU oracle's local deformable-kernel functions (forward and the
three gradients) without importing the reference: against a float64
grid_sample composite with autograd, closed forms, the hat-function identity
and central finite differences."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import _composite as comp
from _cases import make_local, rel_err
from oracle import dk_oracle as orc

CASES = [
    # N, C, H, W, k, S, stride, pad, dil, groups, rot_std
    (2, 4, 7, 6, 3, (4, 4), 1, 1, 1, 1, 0.5),
    (2, 6, 9, 8, 3, (4, 4), 2, 1, 1, 2, 1.0),
    (1, 4, 10, 11, 3, (5, 3), 1, 2, 2, 1, 1.5),
    (2, 6, 8, 8, (5, 3), (7, 4), (1, 2), (2, 0), 1, 3, 0.7),
    (1, 3, 6, 5, 1, (2, 2), 1, 0, 1, 1, 0.6),
    (2, 4, 6, 6, 3, (3, 3), 1, 1, 1, 1, 2.5),   # many samples outside (-1, S)
    (1, 2, 5, 5, 2, (4, 4), 1, 0, 1, 2, 0.5),   # even kernel
]


def _f64(*ts):
    return [t.double() for t in ts]


@pytest.mark.parametrize("case", CASES)
def test_forward_matches_grid_sample_composite(case):
    N, C, H, W, k, S, s, p, d, G, rs = case
    x, wt, rot, gout, cfg = make_local(N, C, H, W, k, S, s, p, d, G, rs, seed=1)
    x, wt, rot = _f64(x, wt, rot)
    want = comp.local_dk(x, rot, wt, **cfg)
    got = orc.sample_depthwise_forward(x.numpy(), rot.numpy(), wt.numpy(), **cfg)
    assert got.shape == tuple(want.shape)
    assert rel_err(got, want) < 1e-12


@pytest.mark.parametrize("case", CASES)
def test_gradients_match_autograd_of_composite(case):
    N, C, H, W, k, S, s, p, d, G, rs = case
    x, wt, rot, gout, cfg = make_local(N, C, H, W, k, S, s, p, d, G, rs, seed=2)
    x, wt, rot, gout = _f64(x, wt, rot, gout)
    xr, wr, rr = x.clone().requires_grad_(), wt.clone().requires_grad_(), rot.clone().requires_grad_()
    comp.local_dk(xr, rr, wr, **cfg).backward(gout)
    gin, grot, gw = orc.sample_depthwise_backward(gout.numpy(), x.numpy(), rot.numpy(), wt.numpy(), **cfg)
    assert rel_err(gin, xr.grad) < 1e-12
    assert rel_err(gw, wr.grad) < 1e-12
    assert rel_err(grot, rr.grad) < 1e-12


def test_scope_equals_kernel_zero_rotation_is_depthwise_conv():
    # centring term (S-k)/2 = 0 and r = 0: taps hit tile cells exactly.
    for (k, s, p, d) in [(3, 1, 1, 1), (3, 2, 1, 1), (3, 1, 2, 2), (5, 1, 2, 1)]:
        x, wt, rot, gout, cfg = make_local(2, 5, 9, 10, k, (k, k), s, p, d, 1, 0.0, seed=3)
        x, wt, rot = _f64(x, wt, rot)
        want = F.conv2d(x, wt, None, s, p, d, groups=5)
        got = orc.sample_depthwise_forward(x.numpy(), rot.numpy(), wt.numpy(), **cfg)
        assert rel_err(got, want) < 1e-13


def test_integer_rotation_shifts_taps():
    # S == k and rotation (dh, dw) = (0, +1) for every tap: tap (f_h, f_w) reads
    # tile cell (f_h, f_w + 1); the last column falls onto the zero outside.
    k = 3
    x, wt, rot, gout, cfg = make_local(1, 3, 6, 6, k, (k, k), 1, 1, 1, 1, 0.0, seed=4)
    x, wt, rot = _f64(x, wt, rot)
    rot[:, 1::2] = 1.0
    shifted = torch.zeros_like(wt)
    shifted[..., :, :-1] = wt[..., :, 1:]
    want = F.conv2d(x, shifted, None, 1, 1, 1, groups=3)
    got = orc.sample_depthwise_forward(x.numpy(), rot.numpy(), wt.numpy(), **cfg)
    assert rel_err(got, want) < 1e-13


def test_tap_and_direction_channel_layout():
    # Move ONE tap of ONE direction by +1 and check only that tap's weight changes:
    # channel (f_h*k_w + f_w)*2 + dir, dir 0 = h (rows), dir 1 = w (columns).
    k = 3
    x, wt, rot, gout, cfg = make_local(1, 2, 5, 5, k, (k, k), 1, 1, 1, 1, 0.0, seed=5)
    x, wt, rot = _f64(x, wt, rot)
    f_h, f_w = 0, 2
    rot[:, (f_h * k + f_w) * 2 + 0] = 1.0  # tap (0,2) now reads tile row 1, column 2
    eff = wt.clone()
    eff[:, 0, f_h, f_w] = wt[:, 0, f_h + 1, f_w]
    want = F.conv2d(x, eff, None, 1, 1, 1, groups=2)
    got = orc.sample_depthwise_forward(x.numpy(), rot.numpy(), wt.numpy(), **cfg)
    assert rel_err(got, want) < 1e-13


def test_group_interleave_c_mod_G():
    # G = 2: group 0 (even channels) unshifted, group 1 (odd channels) shifted by one column.
    k, C, G = 3, 4, 2
    x, wt, rot, gout, cfg = make_local(1, C, 6, 6, k, (k, k), 1, 1, 1, G, 0.0, seed=6)
    x, wt, rot = _f64(x, wt, rot)
    rot[:, k * k * 2 + 1::2] = 1.0  # all w-components of group 1
    eff = wt.clone()
    eff[1::2, :, :, :-1] = wt[1::2, :, :, 1:]
    eff[1::2, :, :, -1] = 0
    want = F.conv2d(x, eff, None, 1, 1, 1, groups=C)
    got = orc.sample_depthwise_forward(x.numpy(), rot.numpy(), wt.numpy(), **cfg)
    assert rel_err(got, want) < 1e-13


def test_everything_outside_scope_is_exact_zero():
    x, wt, rot, gout, cfg = make_local(2, 3, 6, 6, 3, (4, 4), 1, 1, 1, 1, 0.0, seed=7)
    for shift in (-10.0, 10.0, -3.5, 4.0):   # -3.5: coords 0.5-3.5+{0,1,2} <= -1 ; 4.0: >= 4
        r = rot + shift
        out = orc.sample_depthwise_forward(x.numpy(), r.numpy(), wt.numpy(), **cfg)
        gin, grot, gw = orc.sample_depthwise_backward(gout.numpy(), x.numpy(), r.numpy(), wt.numpy(), **cfg)
        for t in (out, gin, grot, gw):
            assert np.count_nonzero(t) == 0


def _hat(t):
    return np.maximum(0.0, 1.0 - np.abs(t))


def test_hat_function_identity_including_borders_and_integers():
    # B(tile, h, w) = sum_ij tile[i, j] * hat(h - i) * hat(w - j): the textbook
    # tensor-product form of zero-extended bilinear interpolation; it needs no floor,
    # so it pins the floor/low-high bookkeeping, the (-1, 0) and (S-1, S) fade bands and
    # integer coordinates.  One output pixel, one tap (k = 1, pad 0), so out = x * B.
    rng = np.random.default_rng(8)
    S = (4, 5)
    tile = rng.standard_normal((1, 1) + S)
    coords = [(-1.0, 2.0), (-0.999, 0.3), (-0.25, -0.75), (0.0, 0.0), (1.0, 2.0), (3.0, 4.0), (3.5, 4.25),
              (3.999, 1.5), (4.0, 1.0), (2.2, 5.0), (2.2, 4.999), (1.5, 1.5), (0.5, 3.75), (-1.0, -1.0)]
    for (h, w) in coords:
        # k = 1: scope coord = 0 + r + (S - 1)/2
        rot = np.array([h - (S[0] - 1) / 2.0, w - (S[1] - 1) / 2.0]).reshape(1, 2, 1, 1)
        x = np.array(2.0).reshape(1, 1, 1, 1)
        got = orc.sample_depthwise_forward(x, rot, tile, kernel_size=1, stride=1, padding=0, dilation=1, groups=1)
        ii, jj = np.arange(S[0]), np.arange(S[1])
        want = 2.0 * (tile[0, 0] * np.outer(_hat(h - ii), _hat(w - jj))).sum()
        assert abs(got.item() - want) < 1e-14, (h, w, got.item(), want)


@pytest.mark.parametrize("case", CASES[:4])
def test_backward_is_the_derivative_of_forward(case):
    N, C, H, W, k, S, s, p, d, G, rs = case
    x, wt, rot, gout, cfg = make_local(N, C, H, W, k, S, s, p, d, G, rs, seed=9)
    x, wt, rot, gout = [t.double().numpy() for t in (x, wt, rot, gout)]
    # keep scope coordinates away from the kinks at integers
    kk = cfg["kernel_size"]
    cen = np.array([(S[0] - kk[0]) / 2.0, (S[1] - kk[1]) / 2.0])
    frac = (rot.reshape(N, -1, 2, *rot.shape[2:]) + cen.reshape(1, 1, 2, 1, 1))
    frac = frac - np.floor(frac)
    bad = (np.minimum(frac, 1 - frac) < 1e-3).reshape(rot.shape)
    rot = rot + 0.01 * bad
    gin, grot, gw = orc.sample_depthwise_backward(gout, x, rot, wt, **cfg)

    def loss(x_, r_, w_):
        return float((orc.sample_depthwise_forward(x_, r_, w_, **cfg) * gout).sum())

    rng = np.random.default_rng(10)
    eps = 1e-6
    for arr, grad, name in ((x, gin, "x"), (rot, grot, "rot"), (wt, gw, "w")):
        for _ in range(12):
            idx = tuple(rng.integers(0, n) for n in arr.shape)
            ap, am = arr.copy(), arr.copy()
            ap[idx] += eps
            am[idx] -= eps
            args_p = {"x": (ap, rot, wt), "rot": (x, ap, wt), "w": (x, rot, ap)}[name]
            args_m = {"x": (am, rot, wt), "rot": (x, am, wt), "w": (x, rot, am)}[name]
            num = (loss(*args_p) - loss(*args_m)) / (2 * eps)
            assert abs(num - grad[idx]) < 1e-6 * max(1.0, abs(num)), (name, idx, num, grad[idx])


def test_linearity_in_input_and_in_weight():
    x, wt, rot, gout, cfg = make_local(2, 4, 7, 7, 3, (4, 4), 1, 1, 1, 1, 1.0, seed=11)
    x2, wt2, _, _, _ = make_local(2, 4, 7, 7, 3, (4, 4), 1, 1, 1, 1, 1.0, seed=12)
    x, wt, rot, x2, wt2 = [t.double().numpy() for t in (x, wt, rot, x2, wt2)]
    f = lambda a, w: orc.sample_depthwise_forward(a, rot, w, **cfg)
    assert rel_err(f(2 * x + 3 * x2, wt), 2 * f(x, wt) + 3 * f(x2, wt)) < 1e-13
    assert rel_err(f(x, 2 * wt - wt2), 2 * f(x, wt) - f(x, wt2)) < 1e-13


def test_float32_oracle_tracks_float64_oracle():
    x, wt, rot, gout, cfg = make_local(2, 8, 12, 12, 3, (4, 4), 1, 1, 1, 1, 1.0, seed=13)
    a32 = [t.numpy() for t in (x, rot, wt)]
    a64 = [t.double().numpy() for t in (x, rot, wt)]
    o32 = orc.sample_depthwise_forward(*a32, **cfg)
    o64 = orc.sample_depthwise_forward(*a64, **cfg)
    assert o32.dtype == np.float32
    assert rel_err(o32, o64) < 1e-6
    g32 = orc.sample_depthwise_backward(gout.numpy(), x.numpy(), rot.numpy(), wt.numpy(), **cfg)
    g64 = orc.sample_depthwise_backward(gout.double().numpy(), x.double().numpy(), rot.double().numpy(),
                                        wt.double().numpy(), **cfg)
    for a, b in zip(g32, g64):
        assert rel_err(a, b) < 1e-5


def test_output_size_rule_matches_conv2d_and_rejects_too_small_input():
    for (H, k, s, p, d) in [(7, 3, 1, 1, 1), (8, 3, 2, 1, 1), (9, 3, 2, 0, 2), (5, 5, 1, 0, 1)]:
        want = F.conv2d(torch.zeros(1, 1, H, H), torch.zeros(1, 1, k, k), None, s, p, d).shape[-1]
        assert orc.output_size(H, k, s, p, d) == want
    with pytest.raises(ValueError):
        orc.make_args((1, 1, 2, 2), (1, 1, 4, 4), 3, 1, 0, 1, 1)
