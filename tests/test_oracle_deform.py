"""Pins the oracle's deformable (kernel-space + image-space offsets) functions:
grid_sample composite with autograd, reduction to the local operator at zero
image offsets, a brute-force depthwise deformable convolution when scope ==
kernel, exact zeros outside the image band, and finite differences."""
import numpy as np
import pytest
import torch

import _composite as comp
from _cases import make_deform, make_local, rel_err
from oracle import dk_oracle as orc

CASES = [
    # N, C, H, W, k, S, stride, pad, dil, groups, rot_std, off_std
    (2, 4, 7, 6, 3, (4, 4), 1, 1, 1, 1, 0.5, 2.0),
    (2, 6, 9, 8, 3, (4, 4), 2, 1, 1, 2, 0.5, 2.0),
    (1, 4, 10, 11, 3, (5, 3), 1, 2, 2, 1, 1.0, 4.0),
    (2, 6, 8, 8, (2, 3), (4, 5), (1, 2), (0, 1), 1, 3, 0.7, 1.0),
    (1, 3, 6, 5, 1, (2, 2), 1, 0, 1, 1, 0.6, 3.0),
]


@pytest.mark.parametrize("case", CASES)
def test_forward_and_gradients_match_composite(case):
    N, C, H, W, k, S, s, p, d, G, rs, os_ = case
    x, wt, rot, off, gout, cfg = make_deform(N, C, H, W, k, S, s, p, d, G, rs, os_, seed=21)
    x, wt, rot, off, gout = [t.double() for t in (x, wt, rot, off, gout)]
    xr, wr, rr, orr = [t.clone().requires_grad_() for t in (x, wt, rot, off)]
    want = comp.deform_dk(xr, orr, rr, wr, **cfg)
    want.backward(gout)
    got = orc.deform_sample_depthwise_forward(x.numpy(), off.numpy(), rot.numpy(), wt.numpy(), **cfg)
    assert rel_err(got, want.detach()) < 1e-12
    gin, goff, grot, gw = orc.deform_sample_depthwise_backward(
        gout.numpy(), x.numpy(), off.numpy(), rot.numpy(), wt.numpy(), **cfg)
    assert rel_err(gin, xr.grad) < 1e-12
    assert rel_err(goff, orr.grad) < 1e-12
    assert rel_err(grot, rr.grad) < 1e-12
    assert rel_err(gw, wr.grad) < 1e-12


def test_zero_image_offset_reduces_to_local_operator():
    x, wt, rot, gout, cfg = make_local(2, 6, 9, 8, 3, (4, 4), 2, 1, 1, 2, 1.0, seed=22)
    x, wt, rot, gout = [t.double().numpy() for t in (x, wt, rot, gout)]
    off = np.zeros((2, 18) + rot.shape[2:])
    a = orc.sample_depthwise_forward(x, rot, wt, **cfg)
    b = orc.deform_sample_depthwise_forward(x, off, rot, wt, **cfg)
    assert rel_err(b, a) < 1e-14
    gin, grot, gw = orc.sample_depthwise_backward(gout, x, rot, wt, **cfg)
    gin2, goff2, grot2, gw2 = orc.deform_sample_depthwise_backward(gout, x, off, rot, wt, **cfg)
    assert rel_err(gin2, gin) < 1e-14
    assert rel_err(grot2, grot) < 1e-14
    assert rel_err(gw2, gw) < 1e-14


def _hat(t):
    return np.maximum(0.0, 1.0 - np.abs(t))


def test_scope_equals_kernel_is_depthwise_deformable_convolution_brute_force():
    # out[n,c,oh,ow] = sum_tap W[c,tap] * sum_{y,x} X[n,c,y,x] hat(ih-y) hat(iw-x): textbook
    # deformable convolution (zero padding), written with hat functions instead of floor.
    N, C, H, W, k = 1, 2, 5, 6, 3
    x, wt, rot, off, gout, cfg = make_deform(N, C, H, W, k, (k, k), 1, 1, 1, 1, 0.0, 1.5, seed=23)
    x, wt, rot, off = [t.double().numpy() for t in (x, wt, rot, off)]
    got = orc.deform_sample_depthwise_forward(x, off, rot, wt, **cfg)
    yy, xx = np.arange(H), np.arange(W)
    want = np.zeros_like(got)
    for c in range(C):
        for oh in range(H):
            for ow in range(W):
                acc = 0.0
                for f_h in range(k):
                    for f_w in range(k):
                        t = f_h * k + f_w
                        ih = oh - 1 + f_h + off[0, 2 * t, oh, ow]
                        iw = ow - 1 + f_w + off[0, 2 * t + 1, oh, ow]
                        acc += wt[c, 0, f_h, f_w] * (x[0, c] * np.outer(_hat(ih - yy), _hat(iw - xx))).sum()
                want[0, c, oh, ow] = acc
    assert rel_err(got, want) < 1e-13


def test_samples_outside_the_image_band_give_exact_zeros():
    x, wt, rot, off, gout, cfg = make_deform(1, 3, 6, 6, 3, (4, 4), 1, 1, 1, 1, 0.3, 0.0, seed=24)
    for shift in (-20.0, 20.0):
        o = off + shift
        out = orc.deform_sample_depthwise_forward(x.numpy(), o.numpy(), rot.numpy(), wt.numpy(), **cfg)
        grads = orc.deform_sample_depthwise_backward(gout.numpy(), x.numpy(), o.numpy(), rot.numpy(),
                                                     wt.numpy(), **cfg)
        for t in (out,) + tuple(grads):
            assert np.count_nonzero(t) == 0


@pytest.mark.parametrize("case", CASES[:3])
def test_backward_is_the_derivative_of_forward(case):
    N, C, H, W, k, S, s, p, d, G, rs, os_ = case
    x, wt, rot, off, gout, cfg = make_deform(N, C, H, W, k, S, s, p, d, G, rs, os_, seed=25)
    x, wt, rot, off, gout = [t.double().numpy() for t in (x, wt, rot, off, gout)]
    # keep both kinds of coordinates away from integer kinks
    kk = cfg["kernel_size"]
    for arr, cen in ((rot, [(S[0] - kk[0]) / 2.0, (S[1] - kk[1]) / 2.0]), (off, [0.0, 0.0])):
        v = arr.reshape(N, -1, 2, *arr.shape[2:]) + np.array(cen).reshape(1, 1, 2, 1, 1)
        fr = v - np.floor(v)
        arr += 0.01 * (np.minimum(fr, 1 - fr) < 1e-3).reshape(arr.shape)
    gin, goff, grot, gw = orc.deform_sample_depthwise_backward(gout, x, off, rot, wt, **cfg)

    def loss(x_, o_, r_, w_):
        return float((orc.deform_sample_depthwise_forward(x_, o_, r_, w_, **cfg) * gout).sum())

    rng = np.random.default_rng(26)
    eps = 1e-6
    base = [x, off, rot, wt]
    for pos, grad in enumerate((gin, goff, grot, gw)):
        for _ in range(10):
            idx = tuple(rng.integers(0, n) for n in base[pos].shape)
            ap = [a.copy() for a in base]
            am = [a.copy() for a in base]
            ap[pos][idx] += eps
            am[pos][idx] -= eps
            num = (loss(*ap) - loss(*am)) / (2 * eps)
            assert abs(num - grad[idx]) < 1e-6 * max(1.0, abs(num)), (pos, idx, num, grad[idx])


def test_float32_oracle_tracks_float64_oracle():
    x, wt, rot, off, gout, cfg = make_deform(2, 8, 12, 12, 3, (4, 4), 2, 1, 1, 1, 0.5, 2.0, seed=27)
    t32 = [t.numpy() for t in (x, off, rot, wt)]
    t64 = [t.double().numpy() for t in (x, off, rot, wt)]
    assert rel_err(orc.deform_sample_depthwise_forward(*t32, **cfg),
                   orc.deform_sample_depthwise_forward(*t64, **cfg)) < 1e-6
    g32 = orc.deform_sample_depthwise_backward(gout.numpy(), *t32, **cfg)
    g64 = orc.deform_sample_depthwise_backward(gout.double().numpy(), *t64, **cfg)
    for a, b in zip(g32, g64):
        assert rel_err(a, b) < 1e-5
