from .backends import dequantize, quantize, quantize_dequantize
from .quantizer import Quantize, QuantizeDequantize

__all__ = ['quantize', 'quantize_dequantize', 'dequantize', 'Quantize', 'QuantizeDequantize']
