"""Autograd Function of the N-d linear sampler.

Same signature and layouts as the reference's ``NdLinearSampleFunction``
(``functions/nd_linear_sample.py:18-62``): ``input`` is ``[C, s_1..s_n]``,
``coord`` is ``[B, n]`` in absolute index units, the result is ``[B, C]``.
The sizes travel to the kernel as host integers (the reference builds a
device tensor per call, ``:22``) and the coordinate gradient comes back already
summed over channels (the reference sums a ``[B, n, C]`` buffer in Python,
``:48-55``).
"""
import torch
from torch.autograd import Function
from torch.autograd.function import once_differentiable

from .. import _lib

__all__ = ['nd_linear_sample']


class NdLinearSampleFunction(Function):
    @staticmethod
    def forward(ctx, input, coord):
        _lib.require_gpu(input, coord)
        if coord.dim() != 2 or coord.size(1) != input.dim() - 1:
            raise ValueError("coord must be [B, %d] for input of shape %s, got %s"
                             % (input.dim() - 1, tuple(input.shape), tuple(coord.shape)))
        input, coord = input.contiguous(), coord.contiguous()
        ctx.save_for_backward(input, coord)
        output = input.new_empty(NdLinearSampleFunction._output_size(input, coord))
        desc = _lib.nd_desc(input, coord)
        L = _lib.lib()
        with torch.cuda.device(input.device):
            # many points per cell: the kernels work on the points sorted by cell; sort once,
            # here, and keep the order for the backward pass
            order = None
            order_bytes = L.dk_nd_linear_sample_order_bytes(desc)
            if order_bytes:
                order = torch.empty(order_bytes, dtype=torch.uint8, device=input.device)
                ws, nbytes = _lib.workspace(L.dk_nd_linear_sample_order_workspace(desc), input.device)
                _lib.check(L.dk_nd_linear_sample_order(desc, _lib.ptr(coord), _lib.ptr(order), _lib.ptr(ws), nbytes,
                                                       _lib.stream_ptr(input)), "nd_linear_sample order")
            ctx.order = order
            ws, nbytes = _lib.workspace(L.dk_nd_linear_sample_forward_workspace(desc), input.device)
            _lib.check(L.dk_nd_linear_sample_forward(
                desc, _lib.ptr(input), _lib.ptr(coord), _lib.ptr(order), _lib.ptr(output), _lib.ptr(ws), nbytes,
                _lib.stream_ptr(input)), "nd_linear_sample forward")
        return output

    @staticmethod
    @once_differentiable  # the kernels are not differentiable a second time: asking for it raises
    def backward(ctx, grad_output):
        input, coord = ctx.saved_tensors
        grad_input = grad_coord = None
        _lib.require_gpu(grad_output, input)
        grad_output = grad_output.contiguous()
        desc = _lib.nd_desc(input, coord)
        L = _lib.lib()
        with torch.cuda.device(input.device):
            s = _lib.stream_ptr(input)
            if ctx.needs_input_grad[0]:
                grad_input = torch.empty_like(input)
                ws, nbytes = _lib.workspace(L.dk_nd_linear_sample_backward_data_workspace(desc), input.device)
                _lib.check(L.dk_nd_linear_sample_backward_data(
                    desc, _lib.ptr(grad_output), _lib.ptr(coord), _lib.ptr(ctx.order), _lib.ptr(grad_input),
                    _lib.ptr(ws), nbytes, s), "nd_linear_sample backward_data")
            if ctx.needs_input_grad[1]:
                grad_coord = torch.zeros_like(coord)
                ws, nbytes = _lib.workspace(L.dk_nd_linear_sample_backward_coord_workspace(desc), input.device)
                _lib.check(L.dk_nd_linear_sample_backward_coord(
                    desc, _lib.ptr(grad_output), _lib.ptr(input), _lib.ptr(coord), _lib.ptr(ctx.order),
                    _lib.ptr(grad_coord), _lib.ptr(ws), nbytes, s), "nd_linear_sample backward_coord")
        return (grad_input, grad_coord)

    @staticmethod
    def _output_size(input, coord):
        output_size = (coord.size(0), input.size(0))
        return output_size


nd_linear_sample = NdLinearSampleFunction.apply
