from .backends import dequantize, quantize, quantize_dequantize
from .encoding import AffineEncoding
from .quantizer import (AffineQuantizerBase, GroupedBlockQuantizeDequantize, MinMaxQuantizer, Quantize,
                        QuantizeDequantize)

__all__ = ['AffineEncoding', 'quantize', 'quantize_dequantize', 'dequantize', 'AffineQuantizerBase', 'MinMaxQuantizer',
           'Quantize', 'QuantizeDequantize', 'GroupedBlockQuantizeDequantize']
