"""The offset branch of ``LocalDeformKernel2d``: its 3x3 ``rotation_conv`` (reference
``modules/deform_kernel.py:165-168``, applied at ``:214``) through the library's kernel for that
shape family where it applies, and through ``torch.nn.functional.conv2d`` everywhere else.

The forward runs on the native kernel (stride 1, padding 1, dilation 1, float32, input channels
a multiple of 16, 18 output channels or at most 16, plane width 7 / 14 / 28 / 56 / 112); the
weight and bias gradients come from kernels of the library as well, the input gradient from
the framework's convolution-backward routine.
"""
import torch
import torch.nn.functional as F
from torch.autograd import Function

from .. import _lib

__all__ = ['offset_conv', 'offset_conv_supported']


def _desc(input, weight):
    return _lib.OffsetConvDesc(input.size(0), input.size(1), weight.size(0), input.size(2), input.size(3),
                               _lib.DK_F32)


def offset_conv_supported(input, weight, bias, stride, padding, dilation, worthwhile=False):
    """Whether the native kernel covers this call; with ``worthwhile`` also whether it is
    expected to be faster than the library convolution."""
    def pair(v):
        return tuple(v) if isinstance(v, (tuple, list)) else (v, v)
    if not (input.is_cuda and input.dtype == torch.float32 and weight.dtype == torch.float32):
        return False
    if input.dim() != 4 or weight.dim() != 4 or tuple(weight.shape[2:]) != (3, 3) or weight.size(1) != input.size(1):
        return False
    if pair(stride) != (1, 1) or pair(padding) != (1, 1) or pair(dilation) != (1, 1):
        return False
    if bias is not None and bias.dtype != torch.float32:
        return False
    if torch.is_autocast_enabled():
        return False
    L = _lib.lib()
    return bool((L.dk_offset_conv_worthwhile if worthwhile else L.dk_offset_conv_supported)(_desc(input, weight)))


class OffsetConvFunction(Function):
    @staticmethod
    def forward(ctx, input, weight, bias):
        input, weight = input.contiguous(), weight.contiguous()
        ctx.save_for_backward(input, weight)
        ctx.has_bias = bias is not None
        b = bias.contiguous() if bias is not None else input.new_zeros(weight.size(0))
        out = input.new_empty(input.size(0), weight.size(0), input.size(2), input.size(3))
        desc = _desc(input, weight)
        L = _lib.lib()
        with torch.cuda.device(input.device):
            ws, nbytes = _lib.workspace(L.dk_offset_conv_forward_workspace(desc), input.device)
            _lib.check(L.dk_offset_conv_forward(desc, _lib.ptr(input), _lib.ptr(weight), _lib.ptr(b),
                                                _lib.ptr(out), _lib.ptr(ws), nbytes, _lib.stream_ptr(input)),
                       "offset_conv forward")
        return out

    @staticmethod
    def backward(ctx, grad_output):
        input, weight = ctx.saved_tensors
        grad_output = grad_output.contiguous()
        gi = gw = gb = None
        if ctx.needs_input_grad[0]:
            gi = torch.nn.grad.conv2d_input(input.shape, weight, grad_output, padding=1)
        if ctx.needs_input_grad[1]:
            gw = torch.empty_like(weight)
            desc = _desc(input, weight)
            L = _lib.lib()
            with torch.cuda.device(input.device):
                ws, nbytes = _lib.workspace(L.dk_offset_conv_backward_weight_workspace(desc), input.device)
                _lib.check(L.dk_offset_conv_backward_weight(desc, _lib.ptr(grad_output), _lib.ptr(input), _lib.ptr(gw),
                                                            _lib.ptr(ws), nbytes, _lib.stream_ptr(input)),
                           "offset_conv weight gradient")
        if ctx.has_bias and ctx.needs_input_grad[2]:
            gb = grad_output.new_empty(weight.size(0))
            desc = _desc(input, weight)
            L = _lib.lib()
            with torch.cuda.device(input.device):
                ws, nbytes = _lib.workspace(L.dk_offset_conv_backward_bias_workspace(desc), input.device)
                _lib.check(L.dk_offset_conv_backward_bias(desc, _lib.ptr(grad_output), _lib.ptr(gb), _lib.ptr(ws),
                                                          nbytes, _lib.stream_ptr(input)), "offset_conv bias gradient")
        return gi, gw, gb


def offset_conv(input, weight, bias=None, stride=1, padding=1, dilation=1, force=False):
    """``F.conv2d(input, weight, bias, stride, padding, dilation)`` for the offset branch: the
    native kernel where it is the faster choice (``force``: wherever it applies)."""
    if offset_conv_supported(input, weight, bias, stride, padding, dilation, worthwhile=not force):
        return OffsetConvFunction.apply(input, weight, bias)
    return F.conv2d(input, weight, bias, stride, padding, dilation)
