"""The convolution ``GlobalDeformKernel2d`` applies with its per-image kernels (reference
``modules/deform_kernel.py:103-111``): ``F.conv2d(x.view(1, n * c, h, w), weight, groups = n * c)``
for a depthwise layer, where ``weight`` holds one ``k x k`` kernel per image and channel.

``image_depthwise_conv(input, weight, stride, padding, dilation)`` takes ``input`` as
``[N, C, H, W]`` and ``weight`` as ``[N * C, 1, k_h, k_w]`` (what ``dynamic_weight`` returns) or
``[N, C, k_h, k_w]`` -- the latter in any dense layout, in particular the permuted view of the
sampler's ``[N * k_h * k_w, C]`` output, which saves the transposing copy of ``:97-101`` and its
gradient -- and returns ``[N, C, H_out, W_out]``: the values and gradients of that grouped
convolution, computed by the library's streaming kernels (forward, input gradient, kernel
gradient; ``include/dk_hip.h``: ``dk_image_depthwise_*``).  GPU tensors only; geometries the
kernels do not cover (``image_depthwise_conv_supported``) are the caller's to route to ``F.conv2d``.
"""
import ctypes

import torch
from torch.autograd import Function
from torch.autograd.function import once_differentiable

from .. import _lib

__all__ = ['image_depthwise_conv', 'image_depthwise_conv_supported']


def _pair(v):
    return tuple(int(e) for e in v) if isinstance(v, (tuple, list)) else (int(v), int(v))


def _desc(input, k_h, k_w, stride, padding, dilation):
    return _lib.ConvDesc(
        input.size(0), input.size(1), input.size(2), input.size(3), k_h, k_w, stride[0], stride[1],
        padding[0], padding[1], dilation[0], dilation[1], 1, 1, 1, _lib.dtype_tag(input), _lib.CLIP_NONE, 0.0, 0.0)


def _check_shapes(input, weight):
    if input.dim() != 4 or weight.dim() != 4:
        raise ValueError("input must be [N, C, H, W] and weight [N * C, 1, k_h, k_w] or [N, C, k_h, k_w]")
    n, c = input.size(0), input.size(1)
    if tuple(weight.shape[:2]) not in ((n * c, 1), (n, c)):
        raise ValueError("weight of shape %s does not hold one kernel per image and channel of an input of shape %s"
                         % (tuple(weight.shape), tuple(input.shape)))


def image_depthwise_conv_supported(input, weight, stride=1, padding=0, dilation=1):
    """Whether the library's kernels cover this call (GPU tensors of one dtype, a geometry whose
    taps fit the kernels' staging area)."""
    if not (input.is_cuda and weight.is_cuda and input.dtype == weight.dtype and input.dtype in _lib._DTYPES):
        return False
    if input.dim() != 4 or weight.dim() != 4:
        return False
    desc = _desc(input, weight.size(2), weight.size(3), _pair(stride), _pair(padding), _pair(dilation))
    return bool(_lib.lib().dk_image_depthwise_supported(desc))


def _dense(t):
    """Whether the tensor's elements occupy numel() distinct consecutive slots in some axis order
    (so that empty_strided with the same strides gives a tensor of the same layout)."""
    expect = 1
    for size, stride in sorted(((sz, st) for sz, st in zip(t.shape, t.stride()) if sz != 1), key=lambda p: p[1]):
        if stride != expect:
            return False
        expect *= size
    return True


def _strides(weight):
    """None for a contiguous kernel tensor, else the C array of its four element strides."""
    if weight.is_contiguous():
        return None
    return (ctypes.c_int64 * 4)(*weight.stride())


class ImageDepthwiseConvFunction(Function):
    @staticmethod
    def forward(ctx, input, weight, stride, padding, dilation):
        _lib.require_gpu(input, weight)
        _check_shapes(input, weight)
        input = input.contiguous()
        if weight.size(1) == 1 and input.size(1) != 1 or not _dense(weight):
            weight = weight.contiguous()  # [N * C, 1, k, k], or a layout with gaps or repeats
        desc = _desc(input, weight.size(2), weight.size(3), stride, padding, dilation)
        L = _lib.lib()
        oh, ow = ctypes.c_int32(0), ctypes.c_int32(0)
        _lib.check(L.dk_conv_out_size(desc, ctypes.byref(oh), ctypes.byref(ow)), "image_depthwise_conv shape")
        out = input.new_empty(input.size(0), input.size(1), oh.value, ow.value)
        with torch.cuda.device(input.device):
            _lib.check(L.dk_image_depthwise_forward(desc, _lib.ptr(input), _lib.ptr(weight), _strides(weight),
                                                    _lib.ptr(out), _lib.stream_ptr(input)),
                       "image_depthwise_conv forward")
        ctx.save_for_backward(input, weight)
        ctx.desc = desc
        return out

    @staticmethod
    @once_differentiable  # the kernels are not differentiable a second time: asking for it raises
    def backward(ctx, grad_output):
        input, weight = ctx.saved_tensors
        grad_output = grad_output.contiguous()
        L = _lib.lib()
        grad_input = grad_weight = None
        with torch.cuda.device(input.device):
            st = _lib.stream_ptr(input)
            if ctx.needs_input_grad[0]:
                grad_input = torch.empty_like(input)
                _lib.check(L.dk_image_depthwise_backward_data(ctx.desc, _lib.ptr(grad_output), _lib.ptr(weight),
                                                              _strides(weight), _lib.ptr(grad_input), st),
                           "image_depthwise_conv grad input")
            if ctx.needs_input_grad[1]:
                # same layout as the kernels: a permuted view of the sampler's output gets a gradient
                # whose rows are the sampler's rows, so no transposing copy runs on the way back either
                grad_weight = torch.empty_strided(weight.shape, weight.stride(), dtype=weight.dtype, device=weight.device)
                _lib.check(L.dk_image_depthwise_backward_weight(ctx.desc, _lib.ptr(grad_output), _lib.ptr(input),
                                                                _lib.ptr(grad_weight), _strides(weight), st),
                           "image_depthwise_conv grad weight")
        return grad_input, grad_weight, None, None, None


def image_depthwise_conv(input, weight, stride=1, padding=0, dilation=1):
    return ImageDepthwiseConvFunction.apply(input, weight, _pair(stride), _pair(padding), _pair(dilation))
