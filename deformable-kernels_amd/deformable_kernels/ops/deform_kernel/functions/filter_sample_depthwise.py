"""Autograd Functions of the depthwise deformable-kernel operators.

Same call signatures, tensor layouts and gradient set as the reference's
``SampleDepthwiseFunction`` and ``DeformableSampleDepthwiseFunction``
(``functions/filter_sample_depthwise.py:19-102`` and ``:105-206``); the bodies
call the C ABI of ``libdk_hip.so`` instead of the CUDA extension.

Differences a user can observe:
  * ``backward`` returns one gradient slot per forward argument (the
    reference returns one too few -- ``:87`` and ``:191`` -- which current
    PyTorch rejects);
  * tensors are validated (device, dtype, shape) and a failing native call
    raises instead of printing;
  * bfloat16 is accepted; fp16/bf16 accumulate in fp32;
  * one optional trailing argument, ``rotation_clip`` (``None``, a ``(min, max)`` pair or
    ``'scope'``): the clamp the reference's module applies to the rotation tensor before the
    call (``modules/deform_kernel.py:185-212``), applied inside the kernels instead;
  * the ``apex.amp.float_function`` wrapper (``:209-211``) is replaced by an
    autocast-aware cast to fp32, apex not being a dependency.
"""
import torch
from torch.autograd import Function
from torch.autograd.function import once_differentiable

from .. import _lib

__all__ = ['sample_depthwise', 'deform_sample_depthwise']


def _output_size(input, kernel_size, stride, padding, dilation):
    # reference functions/filter_sample_depthwise.py:90-102
    output_size = (input.size(0), input.size(1))
    for d in range(input.dim() - 2):
        in_size = input.size(d + 2)
        pad = padding[d]
        kernel = dilation[d] * (kernel_size[d] - 1) + 1
        stride_ = stride[d]
        output_size += ((in_size + (2 * pad) - kernel) // stride_ + 1, )
    if not all(map(lambda s: s > 0, output_size)):
        raise ValueError(
            "convolution input is too small (output would be {})".format(
                'x'.join(map(str, output_size))))
    return output_size


def _check_shapes(input, rotation, weight, out_size, kernel_size, rotation_groups, offset=None):
    if input.dim() != 4 or weight.dim() != 4:
        raise ValueError("input must be [N, C, H, W] and weight [C, 1, S_h, S_w]")
    c = input.size(1)
    if weight.size(0) != c or weight.size(1) != 1:
        raise ValueError("weight must be [C, 1, S_h, S_w] with C = %d, got %s" % (c, tuple(weight.shape)))
    if rotation_groups < 1 or c % rotation_groups != 0:
        raise ValueError("channels (%d) must be divisible by rotation_groups (%d)" % (c, rotation_groups))
    taps2 = kernel_size[0] * kernel_size[1] * 2
    want = (input.size(0), rotation_groups * taps2, out_size[2], out_size[3])
    if rotation is not None and tuple(rotation.shape) != want:
        raise ValueError("rotation must be %s, got %s" % (want, tuple(rotation.shape)))
    if offset is not None:
        want = (input.size(0), taps2, out_size[2], out_size[3])
        if tuple(offset.shape) != want:
            raise ValueError("offset must be %s, got %s" % (want, tuple(offset.shape)))


class SampleDepthwiseFunction(Function):
    @staticmethod
    def forward(
        ctx,
        input,
        rotation,
        weight,
        kernel_size=(3, 3),
        stride=(1, 1),
        padding=(1, 1),
        dilation=(1, 1),
        rotation_groups=1,
        rotation_clip=None,
    ):
        ctx.kernel_size = kernel_size
        ctx.stride = stride
        ctx.padding = padding
        ctx.dilation = dilation
        ctx.rotation_groups = rotation_groups
        ctx.rotation_clip = rotation_clip

        _lib.require_gpu(input, rotation, weight)
        out_size = _output_size(input, kernel_size, stride, padding, dilation)
        _check_shapes(input, rotation, weight, out_size, kernel_size, rotation_groups)
        # A channels-last input runs the library's channels-last kernels and gets a channels-last
        # output (and gradients): no layout change around the operator.  The reference's kernels
        # take planar tensors only.
        # Geometries whose channels-last tables do not fit LDS (e.g. 64 rotation groups) take the planar
        # kernels on a planar copy, and the output goes back to channels-last.
        wants_nhwc = _lib.channels_last(input)
        nhwc = wants_nhwc
        if nhwc:
            probe = _lib.conv_desc(input, weight, kernel_size, stride, padding, dilation, rotation_groups,
                                   rotation_clip, _lib.LAYOUT_NHWC)
            nhwc = _lib.lib().dk_sample_depthwise_layout_supported(probe) == 1
        fmt = torch.channels_last if nhwc else torch.contiguous_format
        ctx.layout = _lib.LAYOUT_NHWC if nhwc else _lib.LAYOUT_NCHW
        input, rotation = input.contiguous(memory_format=fmt), rotation.contiguous(memory_format=fmt)
        weight = weight.contiguous()
        ctx.save_for_backward(input, rotation, weight)
        output = torch.empty(out_size, dtype=input.dtype, device=input.device, memory_format=fmt)
        desc = _lib.conv_desc(input, weight, kernel_size, stride, padding, dilation, rotation_groups,
                              rotation_clip, ctx.layout)
        with torch.cuda.device(input.device):
            _lib.check(_lib.lib().dk_sample_depthwise_forward(
                desc, _lib.ptr(input), _lib.ptr(rotation), _lib.ptr(weight), _lib.ptr(output),
                _lib.stream_ptr(input)), "sample_depthwise forward")
        if wants_nhwc and not nhwc:
            output = output.contiguous(memory_format=torch.channels_last)
        return output

    @staticmethod
    @once_differentiable  # the kernels are not differentiable a second time: asking for it raises
    def backward(ctx, grad_output):
        input, rotation, weight = ctx.saved_tensors
        grad_input = grad_rotation = grad_weight = None
        _lib.require_gpu(grad_output, input)
        nhwc = ctx.layout == _lib.LAYOUT_NHWC
        grad_output = grad_output.contiguous(memory_format=torch.channels_last if nhwc else torch.contiguous_format)
        desc = _lib.conv_desc(input, weight, ctx.kernel_size, ctx.stride, ctx.padding, ctx.dilation,
                              ctx.rotation_groups, ctx.rotation_clip, ctx.layout)
        L = _lib.lib()
        with torch.cuda.device(input.device):
            s = _lib.stream_ptr(input)
            # one native call for the whole backward pass: the gradients that are not needed
            # are passed as NULL and skipped (the reference issues one call per gradient)
            if ctx.needs_input_grad[0]:
                grad_input = torch.empty_like(input)
            if ctx.needs_input_grad[1]:
                grad_rotation = torch.empty_like(rotation)
            ws, nbytes = None, 0
            if ctx.needs_input_grad[2]:
                grad_weight = torch.empty_like(weight)
            if ctx.needs_input_grad[1] or ctx.needs_input_grad[2]:
                ws, nbytes = _lib.workspace(L.dk_sample_depthwise_backward_workspace(desc), input.device)
            _lib.check(L.dk_sample_depthwise_backward(
                desc, _lib.ptr(grad_output), _lib.ptr(input), _lib.ptr(rotation), _lib.ptr(weight),
                _lib.ptr(grad_input), _lib.ptr(grad_rotation), _lib.ptr(grad_weight),
                _lib.ptr(ws), nbytes, s), "sample_depthwise backward")
        return (grad_input, grad_rotation, grad_weight,) + (None,) * 6


class DeformableSampleDepthwiseFunction(Function):
    @staticmethod
    def forward(
        ctx,
        input,
        offset,
        rotation,
        weight,
        kernel_size=(3, 3),
        stride=(1, 1),
        padding=(1, 1),
        dilation=(1, 1),
        rotation_groups=1,
        rotation_clip=None,
    ):
        ctx.kernel_size = kernel_size
        ctx.stride = stride
        ctx.padding = padding
        ctx.dilation = dilation
        ctx.rotation_groups = rotation_groups
        ctx.rotation_clip = rotation_clip

        # rotation = None: no kernel-space offsets (DeformKernelConv2d / DeformConv2d); the library
        # then reads no rotation tensor, where the reference's module hands over a tensor of zeros
        _lib.require_gpu(*(t for t in (input, offset, rotation, weight) if t is not None))
        out_size = _output_size(input, kernel_size, stride, padding, dilation)
        _check_shapes(input, rotation, weight, out_size, kernel_size, rotation_groups, offset)
        input, offset, weight = input.contiguous(), offset.contiguous(), weight.contiguous()
        rotation = rotation.contiguous() if rotation is not None else None
        ctx.save_for_backward(input, offset, rotation, weight)
        output = input.new_empty(out_size)
        desc = _lib.conv_desc(input, weight, kernel_size, stride, padding, dilation, rotation_groups,
                              rotation_clip)
        with torch.cuda.device(input.device):
            _lib.check(_lib.lib().dk_deformable_sample_depthwise_forward(
                desc, _lib.ptr(input), _lib.ptr(offset), _lib.ptr(rotation), _lib.ptr(weight),
                _lib.ptr(output), _lib.stream_ptr(input)), "deform_sample_depthwise forward")
        return output

    @staticmethod
    @once_differentiable  # the kernels are not differentiable a second time: asking for it raises
    def backward(ctx, grad_output):
        input, offset, rotation, weight = ctx.saved_tensors
        grad_input = grad_offset = grad_rotation = grad_weight = None
        _lib.require_gpu(grad_output, input)
        grad_output = grad_output.contiguous()
        desc = _lib.conv_desc(input, weight, ctx.kernel_size, ctx.stride, ctx.padding, ctx.dilation,
                              ctx.rotation_groups, ctx.rotation_clip)
        L = _lib.lib()
        p = _lib.ptr
        with torch.cuda.device(input.device):
            s = _lib.stream_ptr(input)
            if ctx.needs_input_grad[0]:
                grad_input = torch.empty_like(input)
                ws, nbytes = _lib.workspace(
                    L.dk_deformable_sample_depthwise_backward_data_workspace(desc), input.device)
                _lib.check(L.dk_deformable_sample_depthwise_backward_data(
                    desc, p(grad_output), p(offset), p(rotation), p(weight), p(grad_input),
                    p(ws), nbytes, s), "deform_sample_depthwise backward_data")
            both = ctx.needs_input_grad[1] and ctx.needs_input_grad[2] and rotation is not None
            if both:
                # one call for both coordinate gradients (one pass over the input where the library has that kernel)
                grad_offset, grad_rotation = torch.empty_like(offset), torch.empty_like(rotation)
                ws, nbytes = _lib.workspace(
                    L.dk_deformable_sample_depthwise_backward_offset_rotation_workspace(desc), input.device)
                _lib.check(L.dk_deformable_sample_depthwise_backward_offset_rotation(
                    desc, p(grad_output), p(input), p(offset), p(rotation), p(weight),
                    p(grad_offset), p(grad_rotation), p(ws), nbytes, s),
                    "deform_sample_depthwise backward_offset_rotation")
            if ctx.needs_input_grad[1] and not both:
                grad_offset = torch.empty_like(offset)
                ws, nbytes = _lib.workspace(
                    L.dk_deformable_sample_depthwise_backward_offset_workspace(desc), input.device)
                _lib.check(L.dk_deformable_sample_depthwise_backward_offset(
                    desc, p(grad_output), p(input), p(offset), p(rotation), p(weight),
                    p(grad_offset), p(ws), nbytes, s), "deform_sample_depthwise backward_offset")
            if ctx.needs_input_grad[2] and rotation is not None and not both:
                grad_rotation = torch.empty_like(rotation)
                ws, nbytes = _lib.workspace(
                    L.dk_deformable_sample_depthwise_backward_rotation_workspace(desc), input.device)
                _lib.check(L.dk_deformable_sample_depthwise_backward_rotation(
                    desc, p(grad_output), p(input), p(offset), p(rotation), p(weight),
                    p(grad_rotation), p(ws), nbytes, s), "deform_sample_depthwise backward_rotation")
            if ctx.needs_input_grad[3]:
                grad_weight = torch.empty_like(weight)
                ws, nbytes = _lib.workspace(
                    L.dk_deformable_sample_depthwise_backward_filter_workspace(desc), input.device)
                _lib.check(L.dk_deformable_sample_depthwise_backward_filter(
                    desc, p(grad_output), p(input), p(offset), p(rotation), p(grad_weight),
                    p(ws), nbytes, s), "deform_sample_depthwise backward_filter")
        return (grad_input, grad_offset, grad_rotation, grad_weight,) + (None,) * 6


def _float_function(fn):
    """Stand-in for ``apex.amp.float_function`` (reference ``:209-211``): inside an
    autocast region the floating-point tensor arguments are cast to fp32 and the
    op runs with autocast off; outside one it is the identity wrapper."""
    def wrapper(*args):
        if torch.is_autocast_enabled():
            args = tuple(a.float() if torch.is_tensor(a) and a.is_floating_point() else a for a in args)
            with torch.autocast(device_type="cuda", enabled=False):
                return fn(*args)
        return fn(*args)
    wrapper.__wrapped__ = fn
    return wrapper


# register as fp32 functions.
sample_depthwise = _float_function(SampleDepthwiseFunction.apply)
deform_sample_depthwise = _float_function(DeformableSampleDepthwiseFunction.apply)
