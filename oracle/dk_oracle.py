"""TEST INFRASTRUCTURE ONLY -- ctypes/numpy binding of the CPU oracle.

Loads ``oracle/_build/libdk_oracle.so`` (built by ``make -C oracle``) and
exposes one function per reference entry point, operating on numpy arrays in
float32 or float64.  Only ``tests/``, the smoke check and the benchmark's
``cpu_baseline`` leg import this module; the shipped package never does.

The host-side conventions restated here follow the reference's Python and C++
glue: output size (``functions/filter_sample_depthwise.py:90-102``,
``csrc/filter_sample_depthwise_cuda.cpp:42-43``), zero-filled gradient buffers
(``functions/filter_sample_depthwise.py:64,72,80``), ``shape`` passed as a
floating tensor of the data's dtype and ``prod_shape = data.stride(0)``
(``functions/nd_linear_sample.py:22``, ``csrc/nd_linear_sample_cuda.cpp:15-21``)
and the ``sum(2)`` over per-channel coordinate gradients
(``functions/nd_linear_sample.py:48-55``).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libdk_oracle.so")


class _Args(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int) for n in (
        "batch", "channel", "in_h", "in_w", "k_h", "k_w", "stride_h", "stride_w",
        "pad_h", "pad_w", "dil_h", "dil_w", "out_h", "out_w", "scope_h", "scope_w", "groups")]


def build():
    """(Re)build the oracle shared library with gcc."""
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.dko_max_threads.restype = ctypes.c_int
    return _lib


def max_threads():
    return int(lib().dko_max_threads())


def set_threads(n):
    lib().dko_set_threads(ctypes.c_int(int(n)))


def _pair(v):
    return (int(v), int(v)) if np.isscalar(v) else (int(v[0]), int(v[1]))


def _suffix(dtype):
    if dtype == np.float32:
        return "_f32"
    if dtype == np.float64:
        return "_f64"
    raise TypeError("oracle supports float32 and float64 only, got %s" % dtype)


def _c(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def output_size(in_size, kernel, stride, pad, dil):
    return (in_size + 2 * pad - (dil * (kernel - 1) + 1)) // stride + 1


def make_args(x_shape, w_shape, kernel_size, stride, padding, dilation, groups):
    k, s, p, d = _pair(kernel_size), _pair(stride), _pair(padding), _pair(dilation)
    n, c, h, w = (int(v) for v in x_shape)
    oh = output_size(h, k[0], s[0], p[0], d[0])
    ow = output_size(w, k[1], s[1], p[1], d[1])
    if oh <= 0 or ow <= 0:
        raise ValueError("convolution input is too small (output would be %dx%dx%dx%d)" % (n, c, oh, ow))
    return _Args(n, c, h, w, k[0], k[1], s[0], s[1], p[0], p[1], d[0], d[1], oh, ow,
                 int(w_shape[2]), int(w_shape[3]), int(groups))


# --------------------------------------------------------------------------
# local deformable kernel
# --------------------------------------------------------------------------

def sample_depthwise_forward(x, rot, w, kernel_size=(3, 3), stride=(1, 1), padding=(1, 1),
                             dilation=(1, 1), groups=1):
    dt = np.asarray(x).dtype
    sfx = _suffix(dt)
    x, rot, w = _c(x, dt), _c(rot, dt), _c(w, dt)
    a = make_args(x.shape, w.shape, kernel_size, stride, padding, dilation, groups)
    assert rot.shape == (a.batch, a.groups * a.k_h * a.k_w * 2, a.out_h, a.out_w), rot.shape
    out = np.empty((a.batch, a.channel, a.out_h, a.out_w), dtype=dt)
    getattr(lib(), "dko_sample_depthwise_forward" + sfx)(ctypes.byref(a), _p(x), _p(rot), _p(w), _p(out))
    return out


def sample_depthwise_backward(gout, x, rot, w, kernel_size=(3, 3), stride=(1, 1), padding=(1, 1),
                              dilation=(1, 1), groups=1):
    """Returns (grad_input, grad_rotation, grad_weight)."""
    dt = np.asarray(x).dtype
    sfx = _suffix(dt)
    gout, x, rot, w = _c(gout, dt), _c(x, dt), _c(rot, dt), _c(w, dt)
    a = make_args(x.shape, w.shape, kernel_size, stride, padding, dilation, groups)
    assert gout.shape == (a.batch, a.channel, a.out_h, a.out_w)
    gin = np.zeros_like(x)
    grot = np.zeros_like(rot)
    gw = np.zeros_like(w)
    L = lib()
    getattr(L, "dko_sample_depthwise_backward_data" + sfx)(ctypes.byref(a), _p(gout), _p(rot), _p(w), _p(gin))
    getattr(L, "dko_sample_depthwise_backward_rotation" + sfx)(
        ctypes.byref(a), _p(gout), _p(x), _p(rot), _p(w), _p(grot))
    getattr(L, "dko_sample_depthwise_backward_filter" + sfx)(ctypes.byref(a), _p(gout), _p(x), _p(rot), _p(gw))
    return gin, grot, gw


# --------------------------------------------------------------------------
# deformable kernel + image-space offsets
# --------------------------------------------------------------------------

def deform_sample_depthwise_forward(x, off, rot, w, kernel_size=(3, 3), stride=(1, 1),
                                    padding=(1, 1), dilation=(1, 1), groups=1):
    dt = np.asarray(x).dtype
    sfx = _suffix(dt)
    x, off, rot, w = _c(x, dt), _c(off, dt), _c(rot, dt), _c(w, dt)
    a = make_args(x.shape, w.shape, kernel_size, stride, padding, dilation, groups)
    assert off.shape == (a.batch, a.k_h * a.k_w * 2, a.out_h, a.out_w), off.shape
    assert rot.shape == (a.batch, a.groups * a.k_h * a.k_w * 2, a.out_h, a.out_w), rot.shape
    out = np.empty((a.batch, a.channel, a.out_h, a.out_w), dtype=dt)
    getattr(lib(), "dko_deformable_sample_depthwise_forward" + sfx)(
        ctypes.byref(a), _p(x), _p(off), _p(rot), _p(w), _p(out))
    return out


def deform_sample_depthwise_backward(gout, x, off, rot, w, kernel_size=(3, 3), stride=(1, 1),
                                     padding=(1, 1), dilation=(1, 1), groups=1):
    """Returns (grad_input, grad_offset, grad_rotation, grad_weight)."""
    dt = np.asarray(x).dtype
    sfx = _suffix(dt)
    gout, x, off, rot, w = _c(gout, dt), _c(x, dt), _c(off, dt), _c(rot, dt), _c(w, dt)
    a = make_args(x.shape, w.shape, kernel_size, stride, padding, dilation, groups)
    gin = np.zeros_like(x)
    goff = np.zeros_like(off)
    grot = np.zeros_like(rot)
    gw = np.zeros_like(w)
    L = lib()
    pre = "dko_deformable_sample_depthwise_backward_"
    getattr(L, pre + "data" + sfx)(ctypes.byref(a), _p(gout), _p(off), _p(rot), _p(w), _p(gin))
    getattr(L, pre + "offset" + sfx)(ctypes.byref(a), _p(gout), _p(x), _p(off), _p(rot), _p(w), _p(goff))
    getattr(L, pre + "rotation" + sfx)(ctypes.byref(a), _p(gout), _p(x), _p(off), _p(rot), _p(w), _p(grot))
    getattr(L, pre + "filter" + sfx)(ctypes.byref(a), _p(gout), _p(x), _p(off), _p(rot), _p(gw))
    return gin, goff, grot, gw


# --------------------------------------------------------------------------
# N-d linear sample
# --------------------------------------------------------------------------

def _nd_common(data, coord):
    dt = np.asarray(data).dtype
    data, coord = _c(data, dt), _c(coord, dt)
    channel = data.shape[0]
    dims = data.ndim - 1
    prod_shape = int(np.prod(data.shape[1:]))
    batch = coord.shape[0]
    assert coord.shape == (batch, dims), coord.shape
    shape = np.asarray(data.shape[1:], dtype=dt)
    return dt, data, coord, shape, batch, channel, dims, prod_shape


def nd_linear_sample_forward(data, coord):
    dt, data, coord, shape, B, C, n, P = _nd_common(data, coord)
    out = np.empty((B, C), dtype=dt)
    getattr(lib(), "dko_nd_linear_sample_forward" + _suffix(dt))(
        B, C, n, ctypes.c_long(P), _p(data), _p(shape), _p(coord), _p(out))
    return out


def nd_linear_sample_backward(gout, data, coord):
    """Returns (grad_data, grad_coord) with grad_coord summed over channels."""
    dt, data, coord, shape, B, C, n, P = _nd_common(data, coord)
    gout = _c(gout, dt)
    assert gout.shape == (B, C)
    gdata = np.empty_like(data)
    gcoord_c = np.empty((B, n, C), dtype=dt)
    L = lib()
    getattr(L, "dko_nd_linear_sample_backward_data" + _suffix(dt))(
        B, C, n, ctypes.c_long(P), _p(gout), _p(shape), _p(coord), _p(gdata))
    getattr(L, "dko_nd_linear_sample_backward_coord" + _suffix(dt))(
        B, C, n, ctypes.c_long(P), _p(gout), _p(data), _p(shape), _p(coord), _p(gcoord_c))
    return gdata, gcoord_c.sum(2)


# ---- the convolution GlobalDeformKernel2d applies with its sampled kernels ------------------
#
# Reference: modules/deform_kernel.py:103-111, F.conv2d(x.view(1, n * c, h, w), weight, stride,
# padding, dilation, groups = n * c) with weight [n * c, 1, k, k] for a depthwise layer -- the
# framework's grouped cross-correlation; its gradients are the framework's.  Restated in numpy as
# the textbook sums (one shifted, strided slice of the zero-padded plane per tap), in the dtype of
# the arrays handed in.  Pinned in tests/test_oracle_image_conv.py against torch's conv2d and its autograd
# gradients on the CPU in float64 (a library routine), over strides, paddings and dilations.

def _padded(x, k, stride, pad, dil, out):
    """x zero-padded so that every tap of every output position is inside the array."""
    need = [(out[d] - 1) * stride[d] + (k[d] - 1) * dil[d] + 1 for d in (0, 1)]
    hi = [max(need[d] - pad[d] - x.shape[2 + d], 0) for d in (0, 1)]
    return np.pad(x, ((0, 0), (0, 0), (pad[0], hi[0]), (pad[1], hi[1])))


def image_depthwise_forward(x, w, stride=(1, 1), padding=(0, 0), dilation=(1, 1)):
    """x [N, C, H, W], w [N, C, k_h, k_w] (one kernel per image and channel) -> [N, C, Ho, Wo]."""
    stride, padding, dilation = _pair(stride), _pair(padding), _pair(dilation)
    k = w.shape[2:]
    out = [output_size(x.shape[2 + d], k[d], stride[d], padding[d], dilation[d]) for d in (0, 1)]
    xp = _padded(x, k, stride, padding, dilation, out)
    y = np.zeros(x.shape[:2] + tuple(out), dtype=x.dtype)
    for i in range(k[0]):
        for j in range(k[1]):
            r0, c0 = i * dilation[0], j * dilation[1]
            y += w[:, :, i, j, None, None] * xp[:, :, r0:r0 + (out[0] - 1) * stride[0] + 1:stride[0],
                                                c0:c0 + (out[1] - 1) * stride[1] + 1:stride[1]]
    return y


def image_depthwise_backward(gout, x, w, stride=(1, 1), padding=(0, 0), dilation=(1, 1)):
    """Gradients of image_depthwise_forward w.r.t. x and w for the output gradient gout."""
    stride, padding, dilation = _pair(stride), _pair(padding), _pair(dilation)
    k = w.shape[2:]
    out = gout.shape[2:]
    xp = _padded(x, k, stride, padding, dilation, out)
    gxp = np.zeros_like(xp)
    gw = np.zeros_like(w)
    for i in range(k[0]):
        for j in range(k[1]):
            r0, c0 = i * dilation[0], j * dilation[1]
            rows = slice(r0, r0 + (out[0] - 1) * stride[0] + 1, stride[0])
            cols = slice(c0, c0 + (out[1] - 1) * stride[1] + 1, stride[1])
            gw[:, :, i, j] = (gout * xp[:, :, rows, cols]).sum((2, 3))
            gxp[:, :, rows, cols] += w[:, :, i, j, None, None] * gout
    gx = gxp[:, :, padding[0]:padding[0] + x.shape[2], padding[1]:padding[1] + x.shape[3]]
    return np.ascontiguousarray(gx), gw
