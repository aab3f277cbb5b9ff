from .backends import dequantize, quantize, quantize_dequantize
from .quantizer import GroupedBlockQuantizeDequantize, Quantize, QuantizeDequantize

__all__ = ['quantize', 'quantize_dequantize', 'dequantize', 'Quantize', 'QuantizeDequantize',
           'GroupedBlockQuantizeDequantize']
