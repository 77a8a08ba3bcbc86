"""The offset branch of ``LocalDeformKernel2d``: its 3x3 ``rotation_conv`` (reference
``modules/deform_kernel.py:165-168``, applied at ``:214``).

``offset_conv(input, weight, bias, stride, padding, dilation)`` returns what
``torch.nn.functional.conv2d`` returns.  For float32, float16 and bfloat16 GPU tensors (all of one dtype; fp32
sums, results rounded once) with padding 1, dilation 1, input channels a multiple of 16, 18 output channels or
at most 16, on planes 7, 14, 28, 56 or 112 wide (stride 2: input planes 14 to 112 wide) it runs

  * the forward and the input gradient on the library's shift-GEMM kernels on the 16-bit matrix instructions:
    float16 / bfloat16 elements as they are (exact products), float32 elements as bfloat16 (hi, lo) pairs
    (about 3.5e-6 of the result's scale against the float64 convolution),
  * the weight gradient on the library's kernel for the 16-bit matrix instructions (stride 1 and 2, up to 20
    outputs; float32 tensors again as bfloat16 pairs), per-workgroup partial sums added in a fixed order,
  * the bias gradient on the library's reduction kernel for every shape (the framework's
    reduction over (N, H, W) takes 60-230 us on the large planes),
  * everything else -- other shapes, and passes the library reports as covered
    but not worthwhile (too few images to fill the GPU; the float32 input gradient with fewer than 64 channels or
    on 7 x 7 planes) unless ``force=True`` -- on the framework's convolution routines.

float64, CPU tensors, mixed dtypes and autocast regions go to ``F.conv2d`` unchanged.
"""
import torch
import torch.nn.functional as F
from torch.autograd import Function
from torch.autograd.function import once_differentiable

from .. import _lib

__all__ = ['offset_conv', 'offset_conv_supported']


def _pair(v):
    return tuple(int(e) for e in v) if isinstance(v, (tuple, list)) else (int(v), int(v))


def _desc(input, weight, out=None, stride=1):
    h, w = (input.size(2), input.size(3)) if out is None else (out.size(2), out.size(3))
    return _lib.OffsetConvDesc(input.size(0), input.size(1), weight.size(0), h, w, _lib.dtype_tag(input), stride)


_NATIVE_DTYPES = (torch.float32, torch.float16, torch.bfloat16)


def _float32_gpu(input, weight, bias):
    """Tensors the library's kernels take: on the GPU, all float32 or all float16 or all bfloat16."""
    if not (input.is_cuda and weight.is_cuda and input.dtype in _NATIVE_DTYPES and weight.dtype == input.dtype):
        return False
    if bias is not None and not (bias.is_cuda and bias.dtype == input.dtype):
        return False
    return input.dim() == 4 and weight.dim() == 4 and not torch.is_autocast_enabled()


def offset_conv_supported(input, weight, bias, stride, padding, dilation, worthwhile=False):
    """Whether the native forward / weight-gradient kernels cover this call; with ``worthwhile``
    also whether they are expected to be faster than the library convolution."""
    if not _float32_gpu(input, weight, bias):
        return False
    if tuple(weight.shape[2:]) != (3, 3) or weight.size(1) != input.size(1):
        return False
    if _pair(stride) not in ((1, 1), (2, 2)) or _pair(padding) != (1, 1) or _pair(dilation) != (1, 1):
        return False
    L = _lib.lib()
    desc = _desc(input, weight, stride=_pair(stride)[0])   # stride 2: the library answers for the forward alone
    return bool((L.dk_offset_conv_worthwhile if worthwhile else L.dk_offset_conv_supported)(desc))


class OffsetConvFunction(Function):
    @staticmethod
    def forward(ctx, input, weight, bias, stride, padding, dilation, native, forced=False):
        input, weight = input.contiguous(), weight.contiguous()
        ctx.save_for_backward(input, weight)
        ctx.conv = (stride, padding, dilation)
        ctx.native = native
        ctx.forced = forced
        ctx.has_bias = bias is not None
        if not native:
            return F.conv2d(input, weight, bias, stride, padding, dilation)
        b = bias.contiguous() if bias is not None else input.new_zeros(weight.size(0))
        s = stride[0]
        out = input.new_empty(input.size(0), weight.size(0), (input.size(2) - 1) // s + 1, (input.size(3) - 1) // s + 1)
        desc = _desc(input, weight, stride=s)
        L = _lib.lib()
        with torch.cuda.device(input.device):
            ws, nbytes = _lib.workspace(L.dk_offset_conv_forward_workspace(desc), input.device)
            _lib.check(L.dk_offset_conv_forward(desc, _lib.ptr(input), _lib.ptr(weight), _lib.ptr(b),
                                                _lib.ptr(out), _lib.ptr(ws), nbytes, _lib.stream_ptr(input)),
                       "offset_conv forward")
        return out

    @staticmethod
    @once_differentiable  # the kernels are not differentiable a second time: asking for it raises
    def backward(ctx, grad_output):
        input, weight = ctx.saved_tensors
        stride, padding, dilation = ctx.conv
        grad_output = grad_output.contiguous()
        need_input, need_weight = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        gi = gw = gb = None
        L = _lib.lib()
        # a workspace query of 0 says "this pass is not covered"
        desc = _desc(input, weight, stride=stride[0])
        native_weight = need_weight and ctx.native and L.dk_offset_conv_backward_weight_workspace(desc) > 0
        library_weight = need_weight and not native_weight
        native_input = need_input and ctx.native and L.dk_offset_conv_backward_input_workspace(desc) > 0
        if native_input and not ctx.forced and not L.dk_offset_conv_backward_input_worthwhile(desc):
            native_input = False   # covered, but the framework's kernel is the faster one on this shape
        if (need_input and not native_input) or library_weight:
            # the framework's routine, without its bias gradient
            gi, gw_lib, _ = torch.ops.aten.convolution_backward(
                grad_output, input, weight, None, list(stride), list(padding), list(dilation), False, [0, 0], 1,
                [need_input and not native_input, library_weight, False])
            if library_weight:
                gw = gw_lib
        with torch.cuda.device(input.device):
            if native_input:
                gi = torch.empty_like(input)
                ws, nbytes = _lib.workspace(L.dk_offset_conv_backward_input_workspace(desc), input.device)
                _lib.check(L.dk_offset_conv_backward_input(desc, _lib.ptr(grad_output), _lib.ptr(weight), _lib.ptr(gi),
                                                           _lib.ptr(ws), nbytes, _lib.stream_ptr(input)),
                           "offset_conv input gradient")
            if native_weight:
                gw = torch.empty_like(weight)
                ws, nbytes = _lib.workspace(L.dk_offset_conv_backward_weight_workspace(desc), input.device)
                _lib.check(L.dk_offset_conv_backward_weight(desc, _lib.ptr(grad_output), _lib.ptr(input), _lib.ptr(gw),
                                                            _lib.ptr(ws), nbytes, _lib.stream_ptr(input)),
                           "offset_conv weight gradient")
            if ctx.has_bias and ctx.needs_input_grad[2]:
                gb = grad_output.new_empty(weight.size(0))
                desc = _desc(input, weight, grad_output)
                ws, nbytes = _lib.workspace(L.dk_offset_conv_backward_bias_workspace(desc), input.device)
                _lib.check(L.dk_offset_conv_backward_bias(desc, _lib.ptr(grad_output), _lib.ptr(gb), _lib.ptr(ws),
                                                          nbytes, _lib.stream_ptr(input)), "offset_conv bias gradient")
        return gi, gw, gb, None, None, None, None, None


def offset_conv(input, weight, bias=None, stride=1, padding=1, dilation=1, force=False):
    """``F.conv2d(input, weight, bias, stride, padding, dilation)`` for the offset branch (see the
    module docstring for what runs where)."""
    if not _float32_gpu(input, weight, bias):
        return F.conv2d(input, weight, bias, stride, padding, dilation)
    native = offset_conv_supported(input, weight, bias, stride, padding, dilation, worthwhile=not force)
    return OffsetConvFunction.apply(input, weight, bias, _pair(stride), _pair(padding), _pair(dilation), native,
                                    bool(force))
