"""Parameter-holding modules around the two depthwise operators.

Counterparts of the reference's ``SampleDepthwise`` and
``DeformableSampleDepthwise`` (``ops/deform_kernel/modules/filter_sample_depthwise.py:27-115``
and ``:118-206``): same constructor arguments, the scope weight
``weight[C, 1, S_h, S_w]`` under the state-dict key ``weight`` (plus ``bias``
when requested), uniform(+-1/sqrt(k_h*k_w)) initialisation (``:59-66``) and
zero rotation / offset tensors when the caller passes ``None`` (``:68-76``,
``:155-170``).
"""
import math

import torch
import torch.nn as nn
from torch.nn.modules.utils import _pair

from ..functions.filter_sample_depthwise import (
    sample_depthwise,
    deform_sample_depthwise,
)

__all__ = [
    'SampleDepthwise',
    'DeformableSampleDepthwise',
]


class _ScopeDepthwiseBase(nn.Module):
    """Depthwise layer whose per-channel kernel is resampled from a scope tile."""

    def __init__(self, scope_size, in_channels, out_channels, kernel_size=3, stride=1, padding=1,
                 dilation=1, groups=1, rotation_groups=1, bias=False):
        super().__init__()
        if not (in_channels == out_channels and groups == in_channels):
            raise AssertionError("only depthwise layers are supported: in_channels == out_channels == groups")
        if in_channels % rotation_groups != 0:
            raise AssertionError("in_channels must be divisible by rotation_groups")
        self.in_channels = in_channels
        self.scope_size = tuple(scope_size)
        self.kernel_size = _pair(kernel_size)
        self.stride = _pair(stride)
        self.padding = _pair(padding)
        self.dilation = _pair(dilation)
        self.rotation_groups = rotation_groups

        self.weight = nn.Parameter(torch.empty(in_channels, 1, *self.scope_size))
        if bias:
            self.bias = nn.Parameter(torch.empty(in_channels))
        else:
            self.bias = None
        self.reset_parameters()

    def reset_parameters(self):
        bound = 1.0 / math.sqrt(self.kernel_size[0] * self.kernel_size[1])
        with torch.no_grad():
            self.weight.uniform_(-bound, bound)
            if self.bias is not None:
                self.bias.zero_()

    def _spatial_output(self, input):
        dims = []
        for d in range(2):
            span = self.dilation[d] * (self.kernel_size[d] - 1) + 1
            dims.append((input.size(d + 2) + 2 * self.padding[d] - span) // self.stride[d] + 1)
        if min(dims) <= 0:
            raise ValueError("convolution input is too small (output would be {}x{}x{}x{})".format(
                input.size(0), self.weight.size(0), *dims))
        return dims

    def _zeros_per_tap(self, input, sets):
        oh, ow = self._spatial_output(input)
        return input.new_zeros(input.size(0), sets * self.kernel_size[0] * self.kernel_size[1] * 2, oh, ow)

    def _add_bias(self, out):
        if self.bias is not None:
            out = out + self.bias.view(1, self.in_channels, 1, 1)
        return out

    def extra_repr(self):
        s = 'scope_size={}, in_channels={}, kernel_size={}, stride={}'.format(
            self.scope_size, self.in_channels, self.kernel_size, self.stride)
        if self.padding != (0, 0):
            s += ', padding={}'.format(self.padding)
        if self.dilation != (1, 1):
            s += ', dilation={}'.format(self.dilation)
        if self.rotation_groups != 1:
            s += ', rotation_groups={}'.format(self.rotation_groups)
        if self.bias is None:
            s += ', bias=False'
        return s


class SampleDepthwise(_ScopeDepthwiseBase):
    """Local deformable kernel: ``forward(input, rotation=None)``.  ``rotation_clip`` (not in
    the reference) has the operator clamp the offsets itself, see ``sample_depthwise``."""

    def forward(self, input, rotation=None, rotation_clip=None):
        if rotation is None:
            rotation = self._zeros_per_tap(input, self.rotation_groups)
        out = sample_depthwise(
            input, rotation, self.weight, self.kernel_size, self.stride,
            self.padding, self.dilation, self.rotation_groups, rotation_clip)
        return self._add_bias(out)


class DeformableSampleDepthwise(_ScopeDepthwiseBase):
    """Deformable kernel with image-space offsets: ``forward(input, offset=None, rotation=None)``."""

    def forward(self, input, offset=None, rotation=None, rotation_clip=None):
        if offset is None:
            offset = self._zeros_per_tap(input, 1)
        # rotation = None goes to the operator as it is: the library reads no rotation tensor then,
        # where the reference fills one with zeros (:163-168); same values
        out = deform_sample_depthwise(
            input, offset, rotation, self.weight, self.kernel_size,
            self.stride, self.padding, self.dilation, self.rotation_groups, rotation_clip)
        return self._add_bias(out)
