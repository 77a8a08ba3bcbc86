"""User-facing deformable-kernel layers.

Counterparts of the reference's ``modules/deform_kernel.py``: same class names,
constructor signatures, attribute names and state-dict keys
(``weight`` / ``fc.*`` for the global variant, ``rotation_conv.*`` /
``inner_conv.weight`` for the local one, ``offset_conv.*`` /
``inner_conv.weight`` for the conv variant).  ``apex`` is not needed: the
fp32-under-AMP behaviour of ``amp.float_function`` (``:76``) is provided by an
autocast-aware cast.
"""
import torch
from torch import nn

from ..ops.deform_kernel.functions import (
    image_depthwise_conv, image_depthwise_conv_supported, nd_linear_sample, offset_conv, sample_depthwise)
from ..ops.deform_kernel.modules import (
    SampleDepthwise,
    DeformableSampleDepthwise,
)

__all__ = [
    'GlobalDeformKernel2d',
    'LocalDeformKernel2d',
    'DeformKernel2d',
    'DeformKernelConv2d',
]


def _centred_tap_grid(weight_shape, kernel_size, weight_dilate):
    """Scope coordinates of the undeformed taps, (h, w[, extra dims]) per tap in
    tap order: the ``fc_bias`` list of the reference (``:64-74``, ``:188-203``)."""
    start_h = (weight_shape[0] - (kernel_size - 1) * weight_dilate - 1) / 2.0
    start_w = (weight_shape[1] - (kernel_size - 1) * weight_dilate - 1) / 2.0
    grid = []
    for h in range(kernel_size):
        for w in range(kernel_size):
            grid += [start_h + h * weight_dilate, start_w + w * weight_dilate]
            grid += [(extent - 1) / 2.0 for extent in weight_shape[2:]]
    return grid


def _plain_conv(conv):
    """Whether calling ``offset_conv`` on the convolution's parameters is the same as calling the
    module: no forward / pre-forward / backward hooks on it (hook-based weight or spectral
    norm, profilers and quantisation observers rely on the module call) and ordinary zero padding."""
    hooks = (conv._forward_hooks, conv._forward_pre_hooks, conv._backward_hooks,
             getattr(conv, "_backward_pre_hooks", {}))
    return not any(len(h) for h in hooks) and conv.padding_mode == 'zeros' and conv.groups == 1


class GlobalDeformKernel2d(nn.Module):
    """One set of kernel-space offsets per image, predicted from the pooled
    input; the per-image kernels are sampled with ``nd_linear_sample`` and
    applied by one grouped convolution (reference ``:28-118``)."""

    def __init__(self, weight_shape, in_planes, out_planes, kernel_size=1, stride=1, padding=0,
                 dilation=1, groups=1, bias=False):
        super().__init__()
        assert not bias
        assert len(weight_shape) >= 2
        self.kernel_size = kernel_size
        self.weight_shape = weight_shape
        self.weight_dilate = 1
        self.stride = stride
        self.padding = padding
        self.dilation = dilation
        self.out_planes = out_planes
        self.in_planes = in_planes
        self.group = groups

        self.weight = nn.Parameter(torch.empty(out_planes, in_planes // self.group, *self.weight_shape))
        self.fc = nn.Linear(in_planes, kernel_size * kernel_size * len(self.weight_shape))
        self.fc.zero_init = True
        self.fc_bias = _centred_tap_grid(weight_shape, kernel_size, self.weight_dilate)
        # Depthwise layers on the GPU apply the sampled kernels with the library's per-image depthwise
        # convolution (forward, input gradient, kernel gradient as streaming kernels) instead of the
        # framework's convolution with N * C groups (:103-111); same values, same gradients.  Every
        # other configuration, and this one when the flag is cleared, takes the framework's.
        self.native_conv = True
        # Alternative for depthwise layers with a 2-D scope: one call of the fused sample + depthwise
        # operator with the image's rotation broadcast over its pixels, no sampled kernels at all.
        # Off by default: it is the slower route, and it rounds the coordinates (not the sampled
        # kernels) to the input's dtype, so in 16-bit types its results differ from the reference's
        # sequence by more than rounding of the output where a coordinate sits on a cell border.
        self.fused = False
        self.reset_parameters()

    def reset_parameters(self):
        # The reference leaves `weight` uninitialised (torch.Tensor(...), :52-54) for an external
        # initialiser; give it a definite default so a fresh module is usable.
        nn.init.kaiming_normal_(self.weight.view(self.weight.size(0), self.weight.size(1), -1))

    def dynamic_weight(self, x, weight, per_image=False):
        """The kernels sampled for every image: ``[N * out_planes, in_planes / groups, k, k]`` as in
        the reference (:68-101); with ``per_image`` (depthwise layers) the same values as a
        ``[N, C, k, k]`` view of the sampler's output, without the transposing copy of :97-101."""
        if torch.is_autocast_enabled():
            with torch.autocast(device_type="cuda", enabled=False):
                return self._dynamic_weight(x.float(), weight.float(), per_image)
        return self._dynamic_weight(x, weight, per_image)

    def _dynamic_weight(self, x, weight, per_image):
        n, c, h, w = x.shape
        taps = self.kernel_size * self.kernel_size
        kernels = self.out_planes * self.in_planes // self.group
        avg_x = x.reshape(n, c, -1).mean(2)
        centre = torch.tensor(self.fc_bias, dtype=x.dtype, device=x.device).unsqueeze(0)
        coord = self.fc(avg_x) * self.weight_dilate + centre
        # every dimension is clamped with the extent of dimension 0, as in the reference (:83)
        coord = torch.clamp(coord, 0, self.weight_shape[0] - 1)
        sampled = nd_linear_sample(
            weight.reshape(kernels, *self.weight_shape),
            coord.reshape(n * taps, len(self.weight_shape)),
        )
        if per_image:
            return sampled.view(n, self.kernel_size, self.kernel_size, kernels).permute(0, 3, 1, 2)
        return sampled.view(n, taps, kernels).transpose(1, 2).reshape(
            n * self.out_planes, self.in_planes // self.group, self.kernel_size, self.kernel_size)

    def _fusable(self, x):
        return (self.fused and x.is_cuda and len(self.weight_shape) == 2 and self.weight_dilate == 1
                and self.group == self.in_planes == self.out_planes)

    def _forward_fused(self, x):
        n = x.size(0)
        taps = self.kernel_size * self.kernel_size
        centre = torch.tensor(self.fc_bias, dtype=torch.float32, device=x.device).unsqueeze(0)
        with torch.autocast(device_type="cuda", enabled=False):
            pooled = x.float().mean((2, 3))
            coord = nn.functional.linear(pooled, self.fc.weight.float(), self.fc.bias.float()) * self.weight_dilate + centre
            coord = torch.clamp(coord, 0, self.weight_shape[0] - 1)
            # the operator adds the tap's own position and the centring term back (K.cu:338-341)
            rotation = (coord - centre).to(x.dtype)
        size = lambda v: (v, v) if isinstance(v, int) else tuple(v)
        stride, padding, dilation = size(self.stride), size(self.padding), size(self.dilation)
        ho = (x.size(2) + 2 * padding[0] - dilation[0] * (self.kernel_size - 1) - 1) // stride[0] + 1
        wo = (x.size(3) + 2 * padding[1] - dilation[1] * (self.kernel_size - 1) - 1) // stride[1] + 1
        rotation = rotation.view(n, taps * 2, 1, 1).expand(n, taps * 2, ho, wo).contiguous()
        weight = self.weight.to(x.dtype)
        return sample_depthwise(x, rotation, weight, (self.kernel_size, self.kernel_size), stride, padding,
                                dilation, 1)

    def forward(self, x):
        if self._fusable(x):
            return self._forward_fused(x)
        n, c, h, w = x.shape
        # (inside an autocast region the framework's convolution runs, and returns, the autocast dtype; the
        # library's convolution computes in the tensors' own type, so it is only taken outside such regions)
        if (self.native_conv and x.is_cuda and self.group == self.in_planes == self.out_planes
                and not torch.is_autocast_enabled()):
            kernels = self.dynamic_weight(x, self.weight, per_image=True).to(x.dtype)
            if image_depthwise_conv_supported(x, kernels, self.stride, self.padding, self.dilation):
                return image_depthwise_conv(x, kernels, self.stride, self.padding, self.dilation)
            weight = kernels.reshape(n * c, 1, self.kernel_size, self.kernel_size)
        else:
            weight = self.dynamic_weight(x, self.weight).to(x.dtype)
        out = nn.functional.conv2d(
            x.reshape(1, n * c, h, w), weight, stride=self.stride, padding=self.padding,
            dilation=self.dilation, groups=n * self.group)
        return out.view(n, self.out_planes, out.shape[2], out.shape[3])

    def extra_repr(self):
        s = '{}, {}, weight_shape={}, kernel_size={}, stride={}, weight_dilate={}'.format(
            self.in_planes, self.out_planes, self.weight_shape, self.kernel_size, self.stride,
            self.weight_dilate)
        if self.padding != 0:
            s += ', padding={}'.format(self.padding)
        if self.dilation != 1:
            s += ', dilation={}'.format(self.dilation)
        if self.group != 1:
            s += ', group={}'.format(self.group)
        return s


class LocalDeformKernel2d(nn.Module):
    """Per-pixel kernel-space offsets predicted by ``rotation_conv`` and applied
    by the fused sample + depthwise-convolution operator (reference ``:135-221``)."""

    def __init__(self, weight_shape, in_planes, out_planes, kernel_size=1, stride=1, padding=0,
                 dilation=1, groups=1, rotation_groups=1, bias=False, rotation_clip=None):
        super().__init__()
        assert not bias
        assert len(weight_shape) >= 2
        self.kernel_size = kernel_size
        self.weight_shape = weight_shape
        self.weight_dilate = 1
        self.stride = stride
        self.padding = padding
        self.dilation = dilation
        self.out_planes = out_planes
        self.in_planes = in_planes
        self.rotation_groups = rotation_groups
        self.group = groups

        self.rotation_conv = nn.Conv2d(
            in_planes, rotation_groups * kernel_size * kernel_size * 2,
            kernel_size, stride, padding, dilation, bias=True)
        self.rotation_conv.zero_init = True
        self.rotation_clip = rotation_clip
        # True: the operator clamps the offsets itself (same values and gradients as clamping
        # the tensor first, without the extra passes over it); False: the reference's sequence
        self.fused_clip = True
        # True: rotation_conv runs through offset_conv() -- the library's own forward and weight
        # gradient kernels where they are faster (wide planes, float32, stride 1), its bias
        # gradient kernel everywhere; parameters and results are unchanged
        self.native_offset_conv = True

        self.inner_conv = SampleDepthwise(
            weight_shape, in_planes, out_planes, kernel_size=kernel_size, stride=stride,
            padding=padding, dilation=dilation, groups=groups, rotation_groups=rotation_groups,
            bias=bias)

    def _clip_rotation(self, rotation):
        clip = self.rotation_clip
        if isinstance(clip, dict):
            return rotation.clamp(**clip)
        if isinstance(clip, (tuple, list)) and len(clip) == 2:
            # the reference `**`-expands a tuple here (:186-187), which cannot work; read it as (min, max)
            return rotation.clamp(clip[0], clip[1])
        if clip == 'scope':
            centre = rotation.new_tensor(
                _centred_tap_grid(self.weight_shape, self.kernel_size, self.weight_dilate)
            ).repeat(self.rotation_groups)[None, :, None, None]
            coord = (rotation * self.weight_dilate + centre).clamp(0, self.weight_shape[0] - 1)
            return (coord - centre) / self.weight_dilate
        raise NotImplementedError(
            'Expect rotation_clip to be a (min, max) pair, a clamp kwargs dict or "scope", '
            'but get {}'.format(clip))

    def forward(self, x):
        conv = self.rotation_conv
        if self.native_offset_conv and _plain_conv(conv):
            rotation = offset_conv(x, conv.weight, conv.bias, conv.stride, conv.padding, conv.dilation)
        else:
            rotation = conv(x)
        if self.rotation_clip is not None and self.fused_clip and self.weight_dilate == 1 \
                and len(self.weight_shape) == 2:
            clip = self.rotation_clip
            if not (clip == 'scope' or isinstance(clip, dict) or
                    (isinstance(clip, (tuple, list)) and len(clip) == 2)):
                return self.inner_conv(x, self._clip_rotation(rotation))  # raises NotImplementedError
            return self.inner_conv(x, rotation, clip)
        if self.rotation_clip is not None:
            rotation = self._clip_rotation(rotation)
        if self.weight_dilate != 1:
            rotation = rotation * self.weight_dilate
        return self.inner_conv(x, rotation)


# refer to local deformable kernel as the default.
DeformKernel2d = LocalDeformKernel2d


class DeformKernelConv2d(nn.Module):
    """Image-space offsets predicted by ``offset_conv`` feeding the deformable
    sample + depthwise operator; kernel-space offsets stay zero, as in the
    reference (``:228-281``, ``rotation = None`` at ``:278``)."""

    def __init__(self, weight_shape, in_planes, out_planes, kernel_size=1, stride=1, padding=0,
                 dilation=1, groups=1, bias=False, offset_clip=None):
        super().__init__()
        assert not bias
        self.kernel_size = kernel_size
        self.stride = stride
        self.padding = padding
        self.dilation = dilation
        self.out_planes = out_planes
        self.in_planes = in_planes
        self.group = groups

        self.offset_conv = nn.Conv2d(
            in_planes, kernel_size * kernel_size * 2,
            kernel_size, stride, padding, dilation, bias=True)
        self.offset_conv.zero_init = True
        self.offset_clip = offset_clip
        # as in LocalDeformKernel2d: the library's kernels for the offset branch where they apply
        self.native_offset_conv = True

        self.inner_conv = DeformableSampleDepthwise(
            weight_shape, in_planes, out_planes, kernel_size=kernel_size, stride=stride,
            padding=padding, dilation=dilation, groups=groups, bias=bias)

    def forward(self, x):
        conv = self.offset_conv
        if self.native_offset_conv and _plain_conv(conv):
            offset = offset_conv(x, conv.weight, conv.bias, conv.stride, conv.padding, conv.dilation)
        else:
            offset = conv(x)
        if self.offset_clip is not None:
            offset = offset.clamp(**self.offset_clip)
        if self.dilation != 1:
            offset = offset * self.dilation
        return self.inner_conv(x, offset, None)
