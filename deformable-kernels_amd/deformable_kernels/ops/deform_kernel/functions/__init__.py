from .filter_sample_depthwise import (
    sample_depthwise,
    deform_sample_depthwise,
)
from .nd_linear_sample import nd_linear_sample
from .offset_conv import offset_conv, offset_conv_supported
from .image_depthwise_conv import image_depthwise_conv, image_depthwise_conv_supported

__all__ = [
    'sample_depthwise',
    'deform_sample_depthwise',
    'nd_linear_sample',
    'offset_conv',
    'offset_conv_supported',
    'image_depthwise_conv',
    'image_depthwise_conv_supported',
]
