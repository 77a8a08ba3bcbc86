"""Independent float64 restatements of the operators out of library routines.

Every function here is built from ``torch.nn.functional.grid_sample``
(bilinear, zero padding, ``align_corners=True``) and plain tensor slicing, so
autograd supplies all gradients.  They share no code with the C oracle and are
what pins it: grid_sample has the same zero-outside and floor semantics as the
reference's planar_bilinear / deformable_im2col_bilinear.
"""
import torch
import torch.nn.functional as F


def _pair(v):
    return (v, v) if isinstance(v, int) else (int(v[0]), int(v[1]))


def out_size(n, k, s, p, d):
    return (n + 2 * p - (d * (k - 1) + 1)) // s + 1


def _norm(coord, size):
    # absolute index -> grid_sample's [-1, 1] with align_corners=True
    return 2.0 * coord / (size - 1) - 1.0


def scope_weights(w, rot_h, rot_w, f_h, f_w, k, groups, g):
    """B(Wt[c], f_h + r_h + (S_h-k_h)/2, f_w + r_w + (S_w-k_w)/2) for the
    channels c = g, g+G, ... -> [N, C/G, Ho, Wo]."""
    N = rot_h.shape[0]
    S_h, S_w = w.shape[2], w.shape[3]
    ch = f_h + rot_h + (S_h - k[0]) / 2.0
    cw = f_w + rot_w + (S_w - k[1]) / 2.0
    grid = torch.stack([_norm(cw, S_w), _norm(ch, S_h)], dim=-1)  # N,Ho,Wo,2 (x, y)
    tiles = w[g::groups, 0].unsqueeze(0).expand(N, -1, -1, -1)
    return F.grid_sample(tiles, grid, mode="bilinear", padding_mode="zeros", align_corners=True)


def local_dk(x, rot, w, kernel_size=(3, 3), stride=(1, 1), padding=(1, 1), dilation=(1, 1), groups=1):
    k, s, p, d = _pair(kernel_size), _pair(stride), _pair(padding), _pair(dilation)
    N, C, H, W = x.shape
    Ho, Wo = out_size(H, k[0], s[0], p[0], d[0]), out_size(W, k[1], s[1], p[1], d[1])
    xp = F.pad(x, (p[1], p[1], p[0], p[0]))
    out = torch.zeros(N, C, Ho, Wo, dtype=x.dtype)
    kk = k[0] * k[1]
    for f_h in range(k[0]):
        for f_w in range(k[1]):
            h0, w0 = f_h * d[0], f_w * d[1]
            tap = xp[:, :, h0:h0 + (Ho - 1) * s[0] + 1:s[0], w0:w0 + (Wo - 1) * s[1] + 1:s[1]]
            for g in range(groups):
                base = g * kk * 2 + (f_h * k[1] + f_w) * 2
                b = scope_weights(w, rot[:, base], rot[:, base + 1], f_h, f_w, k, groups, g)
                idx = torch.arange(g, C, groups)
                out = out.index_add(1, idx, tap[:, g::groups] * b)
    return out


def deform_dk(x, off, rot, w, kernel_size=(3, 3), stride=(1, 1), padding=(1, 1), dilation=(1, 1),
              groups=1):
    k, s, p, d = _pair(kernel_size), _pair(stride), _pair(padding), _pair(dilation)
    N, C, H, W = x.shape
    Ho, Wo = out_size(H, k[0], s[0], p[0], d[0]), out_size(W, k[1], s[1], p[1], d[1])
    oh = torch.arange(Ho, dtype=x.dtype).view(1, Ho, 1)
    ow = torch.arange(Wo, dtype=x.dtype).view(1, 1, Wo)
    out = torch.zeros(N, C, Ho, Wo, dtype=x.dtype)
    kk = k[0] * k[1]
    for f_h in range(k[0]):
        for f_w in range(k[1]):
            t = f_h * k[1] + f_w
            ih = oh * s[0] - p[0] + f_h * d[0] + off[:, t * 2]
            iw = ow * s[1] - p[1] + f_w * d[1] + off[:, t * 2 + 1]
            grid = torch.stack([_norm(iw, W), _norm(ih, H)], dim=-1)
            tap = F.grid_sample(x, grid, mode="bilinear", padding_mode="zeros", align_corners=True)
            for g in range(groups):
                base = g * kk * 2 + t * 2
                b = scope_weights(w, rot[:, base], rot[:, base + 1], f_h, f_w, k, groups, g)
                idx = torch.arange(g, C, groups)
                out = out.index_add(1, idx, tap[:, g::groups] * b)
    return out


def nd_sample(data, coord):
    """data [C, s1..sn], coord [B, n] in absolute index units -> [B, C]; n in {2, 3}."""
    n = data.dim() - 1
    B = coord.shape[0]
    sizes = data.shape[1:]
    if n == 2:
        grid = torch.stack([_norm(coord[:, 1], sizes[1]), _norm(coord[:, 0], sizes[0])], -1).view(1, B, 1, 2)
        o = F.grid_sample(data.unsqueeze(0), grid, mode="bilinear", padding_mode="zeros", align_corners=True)
        return o.view(data.shape[0], B).t()
    if n == 3:
        grid = torch.stack([_norm(coord[:, 2], sizes[2]), _norm(coord[:, 1], sizes[1]),
                            _norm(coord[:, 0], sizes[0])], -1).view(1, B, 1, 1, 3)
        o = F.grid_sample(data.unsqueeze(0), grid, mode="bilinear", padding_mode="zeros", align_corners=True)
        return o.view(data.shape[0], B).t()
    raise ValueError(n)
