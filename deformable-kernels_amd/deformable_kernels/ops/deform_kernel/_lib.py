"""ctypes binding of ``libdk_hip.so`` (C ABI in ``include/dk_hip.h``).

Takes the place of the reference's two pybind11 extension modules
(``from .. import filter_sample_depthwise_cuda`` --
``functions/filter_sample_depthwise.py:14`` -- and ``nd_linear_sample_cuda`` --
``functions/nd_linear_sample.py:13``).  The library is built in-tree by
``make -C deformable-kernels_amd/csrc``; there is no fallback: if it is
missing or an entry point reports an error, the caller gets an exception.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdk_hip.so")

DK_F32, DK_F16, DK_BF16, DK_F64 = 0, 1, 2, 3
_DTYPES = {torch.float32: DK_F32, torch.float16: DK_F16, torch.bfloat16: DK_BF16, torch.float64: DK_F64}

ND_MAX_DIMS = 8


class ConvDesc(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in (
        "batch", "channel", "in_h", "in_w", "k_h", "k_w", "stride_h", "stride_w",
        "pad_h", "pad_w", "dil_h", "dil_w", "scope_h", "scope_w", "groups", "dtype", "rotation_clip")
    ] + [("clip_min", ctypes.c_float), ("clip_max", ctypes.c_float), ("layout", ctypes.c_int32)]


class NdDesc(ctypes.Structure):
    _fields_ = [("batch", ctypes.c_int64), ("channel", ctypes.c_int32), ("dims", ctypes.c_int32),
                ("shape", ctypes.c_int32 * ND_MAX_DIMS), ("dtype", ctypes.c_int32)]


class OffsetConvDesc(ctypes.Structure):
    # stride: 0 or 1 for stride 1, 2 for the down-sampling layers (forward of 16-bit tensors only)
    _fields_ = [(n, ctypes.c_int32) for n in ("batch", "in_channels", "out_channels", "h", "w", "dtype", "stride")]


class DkError(RuntimeError):
    pass


_P, _SZ = ctypes.c_void_p, ctypes.c_size_t
_I64P = ctypes.POINTER(ctypes.c_int64)
_CD, _ND, _OC = ctypes.POINTER(ConvDesc), ctypes.POINTER(NdDesc), ctypes.POINTER(OffsetConvDesc)

# name -> (restype, argtypes); must list every symbol include/dk_hip.h declares
SIGNATURES = {
    "dk_version": (ctypes.c_int, []),
    "dk_conv_desc_size": (_SZ, []),
    "dk_nd_desc_size": (_SZ, []),
    "dk_offset_conv_desc_size": (_SZ, []),
    "dk_test_switches": (ctypes.c_uint, [ctypes.c_uint]),
    "dk_status_string": (ctypes.c_char_p, [ctypes.c_int]),
    "dk_conv_out_size": (ctypes.c_int, [_CD, ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_int32)]),
    "dk_sample_depthwise_layout_supported": (ctypes.c_int, [_CD]),
    "dk_sample_depthwise_forward": (ctypes.c_int, [_CD, _P, _P, _P, _P, _P]),
    "dk_sample_depthwise_backward_data": (ctypes.c_int, [_CD, _P, _P, _P, _P, _P]),
    "dk_sample_depthwise_backward_filter_workspace": (_SZ, [_CD]),
    "dk_sample_depthwise_backward_filter": (ctypes.c_int, [_CD, _P, _P, _P, _P, _P, _SZ, _P]),
    "dk_sample_depthwise_backward_filter_static": (ctypes.c_int, [_CD, _P, _P, _P, _P, _P]),
    "dk_sample_depthwise_backward_rotation_workspace": (_SZ, [_CD]),
    "dk_sample_depthwise_backward_rotation": (ctypes.c_int, [_CD, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "dk_sample_depthwise_backward_workspace": (_SZ, [_CD]),
    "dk_sample_depthwise_backward": (ctypes.c_int, [_CD, _P, _P, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "dk_deformable_sample_depthwise_forward": (ctypes.c_int, [_CD, _P, _P, _P, _P, _P, _P]),
    "dk_deformable_sample_depthwise_backward_data_workspace": (_SZ, [_CD]),
    "dk_deformable_sample_depthwise_backward_data": (ctypes.c_int, [_CD, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "dk_deformable_sample_depthwise_backward_filter_workspace": (_SZ, [_CD]),
    "dk_deformable_sample_depthwise_backward_filter": (ctypes.c_int, [_CD, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "dk_deformable_sample_depthwise_backward_offset_workspace": (_SZ, [_CD]),
    "dk_deformable_sample_depthwise_backward_offset": (ctypes.c_int, [_CD, _P, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "dk_deformable_sample_depthwise_backward_rotation_workspace": (_SZ, [_CD]),
    "dk_deformable_sample_depthwise_backward_rotation": (ctypes.c_int, [_CD, _P, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "dk_deformable_sample_depthwise_backward_offset_rotation_workspace": (_SZ, [_CD]),
    "dk_deformable_sample_depthwise_backward_offset_rotation": (ctypes.c_int, [_CD, _P, _P, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "dk_nd_linear_sample_forward_workspace": (_SZ, [_ND]),
    "dk_nd_linear_sample_forward": (ctypes.c_int, [_ND, _P, _P, _P, _P, _P, _SZ, _P]),
    "dk_nd_linear_sample_order_bytes": (_SZ, [_ND]),
    "dk_nd_linear_sample_order_workspace": (_SZ, [_ND]),
    "dk_nd_linear_sample_order": (ctypes.c_int, [_ND, _P, _P, _P, _SZ, _P]),
    "dk_nd_linear_sample_backward_data_workspace": (_SZ, [_ND]),
    "dk_nd_linear_sample_backward_data": (ctypes.c_int, [_ND, _P, _P, _P, _P, _P, _SZ, _P]),
    "dk_nd_linear_sample_backward_coord_workspace": (_SZ, [_ND]),
    "dk_nd_linear_sample_backward_coord": (ctypes.c_int, [_ND, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "dk_image_depthwise_supported": (ctypes.c_int, [_CD]),
    "dk_image_depthwise_forward": (ctypes.c_int, [_CD, _P, _P, _I64P, _P, _P]),
    "dk_image_depthwise_backward_data": (ctypes.c_int, [_CD, _P, _P, _I64P, _P, _P]),
    "dk_image_depthwise_backward_weight": (ctypes.c_int, [_CD, _P, _P, _P, _I64P, _P]),
    "dk_offset_conv_supported": (ctypes.c_int, [_OC]),
    "dk_offset_conv_worthwhile": (ctypes.c_int, [_OC]),
    "dk_offset_conv_forward_workspace": (_SZ, [_OC]),
    "dk_offset_conv_forward": (ctypes.c_int, [_OC, _P, _P, _P, _P, _P, _SZ, _P]),
    "dk_offset_conv_backward_weight_workspace": (_SZ, [_OC]),
    "dk_offset_conv_backward_weight": (ctypes.c_int, [_OC, _P, _P, _P, _P, _SZ, _P]),
    "dk_offset_conv_backward_bias_workspace": (_SZ, [_OC]),
    "dk_offset_conv_backward_bias": (ctypes.c_int, [_OC, _P, _P, _P, _SZ, _P]),
    "dk_offset_conv_backward_input_workspace": (_SZ, [_OC]),
    "dk_offset_conv_backward_input_worthwhile": (ctypes.c_int, [_OC]),
    "dk_offset_conv_backward_input": (ctypes.c_int, [_OC, _P, _P, _P, _P, _SZ, _P]),
}

_lib = None


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise DkError(
                "libdk_hip.so not found at %s -- build it with "
                "`make -C deformable-kernels_amd/csrc` (there is no CPU or eager fallback)" % LIB_PATH)
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, args
        # the descriptors are declared twice, here and in include/dk_hip.h: a struct shorter than the
        # library's would be read past its end
        for struct, size_of in ((ConvDesc, handle.dk_conv_desc_size), (NdDesc, handle.dk_nd_desc_size),
                                (OffsetConvDesc, handle.dk_offset_conv_desc_size)):
            if ctypes.sizeof(struct) != size_of():
                raise DkError("%s is %d bytes here and %d in %s (library version %#x): the binding and the "
                              "library are out of step" % (struct.__name__, ctypes.sizeof(struct), size_of(),
                                                           LIB_PATH, handle.dk_version()))
        _lib = handle
    return _lib


def check(status, what):
    if status != 0:
        raise DkError("%s failed: %s (status %d)" % (what, lib().dk_status_string(status).decode(), status))


def dtype_tag(t):
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise TypeError("unsupported dtype %s (float32, float16, bfloat16, float64)" % t.dtype)


def stream_ptr(t):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def require_gpu(*tensors):
    """The operators exist on the GPU only, as in the reference
    (``functions/filter_sample_depthwise.py:43-44``)."""
    for t in tensors:
        if not t.is_cuda:
            raise NotImplementedError("deformable-kernel operators are implemented for GPU tensors only")
    dev, dt = tensors[0].device, tensors[0].dtype
    for t in tensors[1:]:
        if t.device != dev:
            raise ValueError("all tensors must be on the same device")
        if t.dtype != dt:
            raise TypeError("all tensors must have the same dtype (got %s and %s)" % (dt, t.dtype))


def workspace(nbytes, device):
    if nbytes == 0:
        return None, 0
    buf = torch.empty(nbytes, dtype=torch.uint8, device=device)
    return buf, nbytes


TEST_SWITCHES = ("DK_NO_ROWS", "DK_NO_MFMA", "DK_NO_MFMA_S2", "DK_NO_S2_QUADS", "DK_NO_DEFORM_FAST",
                 "DK_NO_DEFORM_CH", "DK_NO_DEFORM_CH_BIG", "DK_NO_DEFORM_MFMA", "DK_NO_ND_BINS", "DK_NO_ND_MFMA",
                 "DK_NO_GATHER_MFMA", "DK_NO_FILTER_SPLIT", "DK_NO_IMAGE_FLAT", "DK_NO_ND_SMALL", "DK_NO_NHWC_MFMA", "DK_FORCE_GATHER_MFMA",
                 "DK_NO_PIXEL_LANES", "DK_FORCE_PIXEL_LANES", "DK_NO_OFFSET_PAIRS", "DK_NO_OFFSET_WGRAD16", "DK_NO_DEFORM_WINDOW", "DK_FORCE_WIN2", "DK_NO_NHWC_STAGED", "DK_FORCE_NHWC_GATHER_MFMA", "DK_NO_IMAGE_PACKED")


class test_switches:
    """Context manager for tests: run the enclosed calls with the named kernel families switched off
    (``dk_test_switches`` in ``include/dk_hip.h``), then restore the previous mask."""

    def __init__(self, *names):
        self.mask = 0
        for n in names:
            self.mask |= 1 << TEST_SWITCHES.index(n)

    def __enter__(self):
        self.before = lib().dk_test_switches(self.mask)
        return self

    def __exit__(self, *exc):
        lib().dk_test_switches(self.before)
        return False


CLIP_NONE, CLIP_ROTATION, CLIP_COORD = 0, 1, 2


def clip_triple(rotation_clip, weight):
    """(mode, min, max) of the descriptor for a module-level ``rotation_clip`` setting:
    ``None``, a ``(min, max)`` pair / ``clamp`` kwargs dict on the offsets, or ``'scope'``
    (scope coordinate kept inside ``[0, scope_h - 1]``, reference ``modules/deform_kernel.py:188-206``)."""
    if rotation_clip is None:
        return (CLIP_NONE, 0.0, 0.0)
    if isinstance(rotation_clip, str):
        if rotation_clip != 'scope':
            raise NotImplementedError("rotation_clip must be a (min, max) pair or 'scope', got %r" % (rotation_clip,))
        return (CLIP_COORD, 0.0, float(weight.size(2) - 1))
    if isinstance(rotation_clip, dict):
        lo, hi = rotation_clip.get('min'), rotation_clip.get('max')
    else:
        lo, hi = rotation_clip
    lo = -float('inf') if lo is None else float(lo)
    hi = float('inf') if hi is None else float(hi)
    return (CLIP_ROTATION, lo, hi)


LAYOUT_NCHW, LAYOUT_NHWC = 0, 1


def channels_last(t):
    """Whether a 4-d tensor is stored channels-last and not also in the default order."""
    return t.dim() == 4 and not t.is_contiguous() and t.is_contiguous(memory_format=torch.channels_last)


def conv_desc(input, weight, kernel_size, stride, padding, dilation, rotation_groups, rotation_clip=None,
              layout=LAYOUT_NCHW):
    mode, lo, hi = clip_triple(rotation_clip, weight)
    return ConvDesc(
        input.size(0), input.size(1), input.size(2), input.size(3),
        int(kernel_size[0]), int(kernel_size[1]), int(stride[0]), int(stride[1]),
        int(padding[0]), int(padding[1]), int(dilation[0]), int(dilation[1]),
        weight.size(2), weight.size(3), int(rotation_groups), dtype_tag(input), mode, lo, hi, layout)


def nd_desc(data, coord):
    dims = data.dim() - 1
    if dims < 1 or dims > ND_MAX_DIMS:
        raise ValueError("nd_linear_sample supports 1..%d sampling dimensions, got %d" % (ND_MAX_DIMS, dims))
    shape = (ctypes.c_int32 * ND_MAX_DIMS)(*(list(data.shape[1:]) + [1] * (ND_MAX_DIMS - dims)))
    return NdDesc(coord.size(0), data.size(0), dims, shape, dtype_tag(data))
