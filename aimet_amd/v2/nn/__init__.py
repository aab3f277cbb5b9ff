"""Quantized modules of the v2 path."""
from .base import (BaseQuantizationMixin, QuantizationMixin, QuantizedConv2d, QuantizedConvTranspose2d, QuantizedLinear,
                   QuantizedReLU)

__all__ = ['BaseQuantizationMixin', 'QuantizationMixin', 'QuantizedLinear', 'QuantizedConv2d',
           'QuantizedConvTranspose2d', 'QuantizedReLU']
