"""Seeded synthetic inputs shared by the oracle tests, the GPU parity tests,
the smoke check and the benchmark.  Generation order is fixed: x, Wt, rot,
[off], gout, all from one torch.Generator seeded with `seed`."""
import math

import torch


def out_size(n, k, s, p, d):
    return (n + 2 * p - (d * (k - 1) + 1)) // s + 1


def make_local(N, C, H, W, k=3, S=(4, 4), stride=1, pad=1, dil=1, groups=1, rot_std=0.5, seed=0,
               dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    kh, kw = (k, k) if isinstance(k, int) else k
    sh, sw = (stride, stride) if isinstance(stride, int) else stride
    ph, pw = (pad, pad) if isinstance(pad, int) else pad
    dh, dw = (dil, dil) if isinstance(dil, int) else dil
    Ho, Wo = out_size(H, kh, sh, ph, dh), out_size(W, kw, sw, pw, dw)
    x = torch.randn(N, C, H, W, generator=g)
    wt = torch.randn(C, 1, S[0], S[1], generator=g) * math.sqrt(2.0 / (S[0] * S[1]))  # kaiming-normal, fan_in = S_h*S_w
    rot = torch.randn(N, groups * kh * kw * 2, Ho, Wo, generator=g) * rot_std
    gout = torch.randn(N, C, Ho, Wo, generator=g)
    cfg = dict(kernel_size=(kh, kw), stride=(sh, sw), padding=(ph, pw), dilation=(dh, dw), groups=groups)
    return x.to(dtype), wt.to(dtype), rot.to(dtype), gout.to(dtype), cfg


def make_deform(N, C, H, W, k=3, S=(4, 4), stride=1, pad=1, dil=1, groups=1, rot_std=0.5, off_std=2.0,
                seed=0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    kh, kw = (k, k) if isinstance(k, int) else k
    sh, sw = (stride, stride) if isinstance(stride, int) else stride
    ph, pw = (pad, pad) if isinstance(pad, int) else pad
    dh, dw = (dil, dil) if isinstance(dil, int) else dil
    Ho, Wo = out_size(H, kh, sh, ph, dh), out_size(W, kw, sw, pw, dw)
    x = torch.randn(N, C, H, W, generator=g)
    wt = torch.randn(C, 1, S[0], S[1], generator=g) * math.sqrt(2.0 / (S[0] * S[1]))
    rot = torch.randn(N, groups * kh * kw * 2, Ho, Wo, generator=g) * rot_std
    off = torch.randn(N, kh * kw * 2, Ho, Wo, generator=g) * off_std
    gout = torch.randn(N, C, Ho, Wo, generator=g)
    cfg = dict(kernel_size=(kh, kw), stride=(sh, sw), padding=(ph, pw), dilation=(dh, dw), groups=groups)
    return x.to(dtype), wt.to(dtype), rot.to(dtype), off.to(dtype), gout.to(dtype), cfg


def rel_err(a, b):
    """max |a-b| over max |b|: error relative to the scale of the expected tensor."""
    a = torch.as_tensor(a).detach().to(torch.float64)
    b = torch.as_tensor(b).detach().to(torch.float64)
    if b.numel() == 0:
        return 0.0
    scale = float(b.abs().max())
    if scale == 0.0:
        return float((a - b).abs().max())
    return float((a - b).abs().max()) / scale


def mixed_err(a, b):
    """max over the elements of |a - b| / (max|b| + |b|): `mixed_err(a, b) < tol` says that every
    element is within tol * max|b| + tol * |b| of the expected one -- the absolute part bounds the
    elements that are small by cancellation, the relative part scales with the element itself."""
    a = torch.as_tensor(a).detach().to(torch.float64)
    b = torch.as_tensor(b).detach().to(torch.float64)
    if b.numel() == 0:
        return 0.0
    scale = float(b.abs().max())
    if scale == 0.0:
        return float((a - b).abs().max())
    return float(((a - b).abs() / (scale + b.abs())).max())


def elem_err(a, b, eps):
    """max over the elements of |a - b| / (|b| + eps * max|b|): `elem_err(a, b, eps) < tol` says that EVERY element
    is within tol of its own magnitude, with an absolute floor of tol * eps * max|b| for the elements that are small
    by cancellation (their error is set by the terms that cancelled, not by their own size).  With eps << 1 this is
    much tighter than rel_err() on the small elements and the same on the large ones."""
    a = torch.as_tensor(a).detach().to(torch.float64)
    b = torch.as_tensor(b).detach().to(torch.float64)
    if b.numel() == 0:
        return 0.0
    scale = float(b.abs().max())
    if scale == 0.0:
        return float((a - b).abs().max())
    return float(((a - b).abs() / (b.abs() + eps * scale)).max())


def clipped_rotation(rot, clip, kernel_size, scope, groups):
    """What the reference's module does to the rotation tensor before the operator
    (modules/deform_kernel.py:185-212), restated on torch CPU tensors in the tensor's own
    precision: returns (clamped rotation, mask of the entries that were NOT clamped)."""
    if clip == 'scope':
        kh, kw = kernel_size
        bias = []
        for h in range(kh):
            for w in range(kw):
                bias += [(scope[0] - (kh - 1) - 1) / 2.0 + h, (scope[1] - (kw - 1) - 1) / 2.0 + w]
        bias = torch.tensor(bias, dtype=rot.dtype).repeat(groups)[None, :, None, None]
        coord = rot + bias
        open_ = (coord >= 0) & (coord <= scope[0] - 1)
        return coord.clamp(0, scope[0] - 1) - bias, open_
    lo, hi = clip
    return rot.clamp(lo, hi), (rot >= lo) & (rot <= hi)
