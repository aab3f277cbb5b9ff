from .backends import dequantize, quantize, quantize_dequantize
from .encoding import AffineEncoding
from .quantizer import GroupedBlockQuantizeDequantize, Quantize, QuantizeDequantize

__all__ = ['AffineEncoding', 'quantize', 'quantize_dequantize', 'dequantize', 'Quantize', 'QuantizeDequantize',
           'GroupedBlockQuantizeDequantize']
